// Row-wise losses with fused backward: KD soft-target (plain and row-masked,
// any row width) and BYOL normalised MSE.  A "group" of threads owns one row:
// a single 64-wide wavefront for narrow rows, a whole workgroup for wide
// (vocabulary-sized) rows.  All accumulation is fp32; storage is fp32, bf16
// or fp16.
#include "common.h"

namespace ts {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -3.0e38f;  // finite stand-in for -inf: keeps exp2(m_old - m_new) NaN-free

// Online soft-max state of part of a row, in the log2 domain:
//   m = running maximum, z = sum 2^(x-m), a = sum 2^(x-m) * w  (w: a weight
//   carried along, here x_teacher - x_student).
struct RowStat {
  float m, z, a;
};

__device__ __forceinline__ RowStat stat_init() { return RowStat{kNegBig, 0.f, 0.f}; }

__device__ __forceinline__ RowStat stat_merge(RowStat p, RowStat q) {
  const float m = fmaxf(p.m, q.m);
  const float rp = exp2f(p.m - m), rq = exp2f(q.m - m);
  return RowStat{m, p.z * rp + q.z * rq, p.a * rp + q.a * rq};
}

__device__ __forceinline__ RowStat stat_wave_reduce(RowStat s) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    RowStat o{__shfl_xor(s.m, off, kWave), __shfl_xor(s.z, off, kWave), __shfl_xor(s.a, off, kWave)};
    s = stat_merge(s, o);
  }
  return s;
}

// Folds VEC elements into the teacher (with weight) and student states: one
// rescale per state per VEC elements instead of one per element.
template <int VEC>
__device__ __forceinline__ void stat_update(RowStat& st, RowStat& ss, const float (&xt)[VEC],
                                            const float (&xs)[VEC]) {
  float mt = xt[0], ms = xs[0];
#pragma unroll
  for (int i = 1; i < VEC; ++i) {
    mt = fmaxf(mt, xt[i]);
    ms = fmaxf(ms, xs[i]);
  }
  const float nmt = fmaxf(st.m, mt), nms = fmaxf(ss.m, ms);
  const float rt = exp2f(st.m - nmt), rs = exp2f(ss.m - nms);
  float zt = st.z * rt, at = st.a * rt, zs = ss.z * rs;
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    const float et = exp2f(xt[i] - nmt);
    zt += et;
    at += et * (xt[i] - xs[i]);
    zs += exp2f(xs[i] - nms);
  }
  st = RowStat{nmt, zt, at};
  ss = RowStat{nms, zs, 0.f};
}

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
__device__ __forceinline__ void store16(T* p, const Vec16<T>& v) {
  u32x4 raw;
  __builtin_memcpy(&raw, &v, 16);
  *reinterpret_cast<u32x4*>(p) = raw;
}

// One group of GROUP threads per row; BLOCK/GROUP rows per workgroup.
//   pass 1: one sweep over both rows -> (max, sum-exp, weighted sum) of the
//           teacher row and (max, sum-exp) of the student row, online.
//   pass 2: second sweep (L2-resident: the group just read these lines) ->
//           grad = g * (q - p).
// Rows with mask == 0 only zero their gradient row.
template <typename T, int BLOCK, int GROUP>
__global__ __launch_bounds__(BLOCK) void kd_rows_kernel(
    const T* __restrict__ s, const T* __restrict__ t, const uint8_t* __restrict__ mask,
    const int* __restrict__ n_sel_dev, int64_t n_rows, int64_t V, int64_t ld_s, int64_t ld_t,
    int64_t ld_g, float kscale /* inv_T * log2(e) */, float gscale /* loss_scale * inv_T */,
    float* __restrict__ row_loss, T* __restrict__ grad) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int NW = GROUP / kWave;  // wavefronts per group
  __shared__ RowStat lds_t[BLOCK / kWave];
  __shared__ RowStat lds_s[BLOCK / kWave];

  const int gtid = threadIdx.x % GROUP;
  const int64_t row = (int64_t)blockIdx.x * (BLOCK / GROUP) + threadIdx.x / GROUP;
  const bool row_ok = row < n_rows;
  // With GROUP == BLOCK the whole workgroup shares one row, so early exits
  // below are uniform; with GROUP == kWave each wavefront exits on its own and
  // never reaches a __syncthreads (NW == 1 uses none).
  if (!row_ok) return;

  const T* srow = s + row * ld_s;
  const T* trow = t + row * ld_t;
  T* grow = grad ? grad + row * ld_g : nullptr;

  const bool selected = mask ? (mask[row] != 0) : true;

  // Common misalignment of the three rows (elements before the first 16-byte
  // boundary); -1 when they disagree and the scalar path must be used.
  const uint32_t mis_s = (uint32_t)((uintptr_t)srow & 15u), mis_t = (uint32_t)((uintptr_t)trow & 15u);
  const uint32_t mis_g = grow ? (uint32_t)((uintptr_t)grow & 15u) : mis_s;
  const bool vec_ok = (mis_s == mis_t) && (mis_s == mis_g);
  int64_t head = vec_ok ? (int64_t)(((16u - mis_s) & 15u) / sizeof(T)) : V;
  if (head > V) head = V;
  const int64_t nvec = (V - head) / VEC;
  const int64_t tail0 = head + nvec * VEC;  // first tail element

  if (!selected) {
    if (gtid == 0) row_loss[row] = 0.f;
    if (grow) {
      const T zero = from_f32<T>(0.f);
      Vec16<T> z;
#pragma unroll
      for (int i = 0; i < VEC; ++i) z.v[i] = zero;
      for (int64_t i = gtid; i < head; i += GROUP) grow[i] = zero;
      for (int64_t v = gtid; v < nvec; v += GROUP) store16(grow + head + v * VEC, z);
      for (int64_t i = tail0 + gtid; i < V; i += GROUP) grow[i] = zero;
    }
    return;
  }

  RowStat st = stat_init(), ss = stat_init();
  {
    float xt1[1], xs1[1];
    for (int64_t i = gtid; i < head; i += GROUP) {
      xt1[0] = to_f32(trow[i]) * kscale;
      xs1[0] = to_f32(srow[i]) * kscale;
      stat_update<1>(st, ss, xt1, xs1);
    }
    for (int64_t v = gtid; v < nvec; v += GROUP) {
      const Vec16<T> vt = load16(trow + head + v * VEC);
      const Vec16<T> vs = load16(srow + head + v * VEC);
      float xt[VEC], xs[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        xt[i] = to_f32(vt.v[i]) * kscale;
        xs[i] = to_f32(vs.v[i]) * kscale;
      }
      stat_update<VEC>(st, ss, xt, xs);
    }
    for (int64_t i = tail0 + gtid; i < V; i += GROUP) {
      xt1[0] = to_f32(trow[i]) * kscale;
      xs1[0] = to_f32(srow[i]) * kscale;
      stat_update<1>(st, ss, xt1, xs1);
    }
  }

  st = stat_wave_reduce(st);
  ss = stat_wave_reduce(ss);
  if (NW > 1) {
    const int w = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) {
      lds_t[w] = st;
      lds_s[w] = ss;
    }
    __syncthreads();
    st = lds_t[0];
    ss = lds_s[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) {
      st = stat_merge(st, lds_t[i]);
      ss = stat_merge(ss, lds_s[i]);
    }
  }

  const float lse_t = st.m + log2f(st.z);  // log2 sum 2^x over the teacher row
  const float lse_s = ss.m + log2f(ss.z);
  if (gtid == 0) row_loss[row] = kLn2 * (st.a / st.z - lse_t + lse_s);

  if (!grow) return;
  const float B = n_sel_dev ? (float)(*n_sel_dev) : (float)n_rows;
  const float g = gscale / B;

  for (int64_t i = gtid; i < head; i += GROUP) {
    const float p = exp2f(to_f32(trow[i]) * kscale - lse_t);
    const float q = exp2f(to_f32(srow[i]) * kscale - lse_s);
    grow[i] = from_f32<T>(g * (q - p));
  }
  for (int64_t v = gtid; v < nvec; v += GROUP) {
    const Vec16<T> vt = load16(trow + head + v * VEC);
    const Vec16<T> vs = load16(srow + head + v * VEC);
    Vec16<T> o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float p = exp2f(to_f32(vt.v[i]) * kscale - lse_t);
      const float q = exp2f(to_f32(vs.v[i]) * kscale - lse_s);
      o.v[i] = from_f32<T>(g * (q - p));
    }
    store16(grow + head + v * VEC, o);
  }
  for (int64_t i = tail0 + gtid; i < V; i += GROUP) {
    const float p = exp2f(to_f32(trow[i]) * kscale - lse_t);
    const float q = exp2f(to_f32(srow[i]) * kscale - lse_s);
    grow[i] = from_f32<T>(g * (q - p));
  }
}

// n_sel = number of non-zero mask bytes.  One workgroup.
__global__ __launch_bounds__(1024) void mask_count_kernel(const uint8_t* __restrict__ mask,
                                                          int64_t n, int* __restrict__ out) {
  __shared__ float lds[1024 / kWave];
  int c = 0;
  for (int64_t i = threadIdx.x; i < n; i += 1024) c += mask[i] != 0;
  // counts are < 2^24 per partial for any n_rows the launcher accepts, so
  // the float sum is exact
  const float tot = block_sum<1024 / kWave>((float)c, lds);
  if (threadIdx.x == 0) *out = (int)tot;
}

// out = scale * sum(v[0..n)) / denom, summed in a fixed order (deterministic).
__global__ __launch_bounds__(1024) void sum_scale_kernel(const float* __restrict__ v, int64_t n,
                                                         float scale, const int* __restrict__ denom_dev,
                                                         float denom, float* __restrict__ out) {
  __shared__ float lds[1024 / kWave];
  float acc = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += 1024) acc += v[i];
  const float tot = block_sum<1024 / kWave>(acc, lds);
  if (threadIdx.x == 0) {
    const float d = denom_dev ? (float)(*denom_dev) : denom;
    *out = scale * (tot / d);
  }
}

// grad[r, :] *= *g, skipped entirely when *g == 1.
template <typename T>
__global__ __launch_bounds__(256) void scale_rows_kernel(T* __restrict__ grad, int64_t V, int64_t ld,
                                                         const float* __restrict__ g_dev) {
  const float g = *g_dev;
  if (g == 1.0f) return;
  T* row = grad + (int64_t)blockIdx.y * ld;
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int64_t i = i0 + k;
    if (i < V) row[i] = from_f32<T>(to_f32(row[i]) * g);
  }
}

// ---- BYOL ---------------------------------------------------------------
// One wavefront per (pair, row).  x^ = x / max(|x|, eps) as F.normalize does.
template <typename T>
__global__ __launch_bounds__(256) void byol_rows_kernel(const T* __restrict__ x1, const T* __restrict__ y1,
                                                        const T* __restrict__ x2, const T* __restrict__ y2,
                                                        int64_t n, int64_t c, float* __restrict__ row_loss,
                                                        T* __restrict__ gx1, T* __restrict__ gx2) {
  constexpr float kEps = 1e-12f;
  const int lane = threadIdx.x % kWave;
  const int64_t vrow = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int64_t total = x2 ? 2 * n : n;
  if (vrow >= total) return;
  const bool second = vrow >= n;
  const int64_t row = second ? vrow - n : vrow;
  const T* x = (second ? x2 : x1) + row * c;
  const T* y = (second ? y2 : y1) + row * c;
  T* gx = second ? gx2 : gx1;
  if (gx) gx += row * c;

  float sxx = 0.f, syy = 0.f, sxy = 0.f;
  for (int64_t i = lane; i < c; i += kWave) {
    const float a = to_f32(x[i]), b = to_f32(y[i]);
    sxx += a * a;
    syy += b * b;
    sxy += a * b;
  }
  sxx = wave_sum(sxx);
  syy = wave_sum(syy);
  sxy = wave_sum(sxy);
  const float nx = sqrtf(sxx), ny = sqrtf(syy);
  const float dx = fmaxf(nx, kEps), dy = fmaxf(ny, kEps);
  const float cosv = sxy / (dx * dy);
  if (lane == 0) row_loss[vrow] = 2.f - 2.f * cosv;
  if (!gx) return;
  // d/dx of -2 <x/dx, y/dy> / n, with dx = |x| (or the constant eps below it).
  const float k = -2.f / (float)n;
  const float proj = (nx >= kEps) ? cosv / dx : 0.f;  // (x^ . y^) / dx, zero once the norm is clamped
  for (int64_t i = lane; i < c; i += kWave) {
    const float a = to_f32(x[i]), b = to_f32(y[i]);
    gx[i] = from_f32<T>(k * (b / (dx * dy) - proj * (a / dx)));
  }
}

template <typename T>
int launch_kd(const void* s, const void* t, const uint8_t* mask, int64_t n_rows, int64_t V,
              int64_t ld_s, int64_t ld_t, float inv_T, float loss_scale, void* ws, float* loss_out,
              void* grad, int64_t ld_g, hipStream_t stream) {
  int* n_sel = reinterpret_cast<int*>(ws);
  float* row_loss = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + 16);
  if (mask) {
    hipLaunchKernelGGL(mask_count_kernel, dim3(1), dim3(1024), 0, stream, mask, n_rows, n_sel);
    int rc = check_launch();
    if (rc) return rc;
  }
  const int* n_sel_arg = mask ? n_sel : nullptr;
  const float kscale = inv_T * kLog2e, gscale = loss_scale * inv_T;
  const T* sp = reinterpret_cast<const T*>(s);
  const T* tp = reinterpret_cast<const T*>(t);
  T* gp = reinterpret_cast<T*>(grad);
  if (V <= 2048) {
    constexpr int BLOCK = 256, GROUP = kWave;
    const int64_t blocks = (n_rows + (BLOCK / GROUP) - 1) / (BLOCK / GROUP);
    hipLaunchKernelGGL((kd_rows_kernel<T, BLOCK, GROUP>), dim3((unsigned)blocks), dim3(BLOCK), 0,
                       stream, sp, tp, mask, n_sel_arg, n_rows, V, ld_s, ld_t, ld_g, kscale, gscale,
                       row_loss, gp);
  } else {
    constexpr int BLOCK = 512, GROUP = 512;
    hipLaunchKernelGGL((kd_rows_kernel<T, BLOCK, GROUP>), dim3((unsigned)n_rows), dim3(BLOCK), 0,
                       stream, sp, tp, mask, n_sel_arg, n_rows, V, ld_s, ld_t, ld_g, kscale, gscale,
                       row_loss, gp);
  }
  int rc = check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(sum_scale_kernel, dim3(1), dim3(1024), 0, stream, row_loss, n_rows, loss_scale,
                     n_sel_arg, (float)n_rows, loss_out);
  return check_launch();
}

template <typename T>
int launch_byol(const void* x1, const void* y1, const void* x2, const void* y2, int64_t n, int64_t c,
                float* ws, float* loss_out, void* gx1, void* gx2, hipStream_t stream) {
  const int64_t total = x2 ? 2 * n : n;
  const int64_t blocks = (total + 3) / 4;
  hipLaunchKernelGGL((byol_rows_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                     (const T*)x1, (const T*)y1, (const T*)x2, (const T*)y2, n, c, ws, (T*)gx1,
                     (T*)gx2);
  int rc = check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(sum_scale_kernel, dim3(1), dim3(1024), 0, stream, ws, total, 1.0f,
                     (const int*)nullptr, (float)n, loss_out);
  return check_launch();
}

inline size_t dtype_size(int dtype) { return dtype == TS_F32 ? 4 : 2; }

// out = scale * sum(v[0..n)) / denom on one workgroup (shared with infonce.hip)
int launch_sum_scale(const float* v, int64_t n, float scale, float denom, float* out, hipStream_t stream) {
  hipLaunchKernelGGL(sum_scale_kernel, dim3(1), dim3(1024), 0, stream, v, n, scale, (const int*)nullptr, denom,
                     out);
  return check_launch();
}

}  // namespace ts

extern "C" {

size_t ts_kd_workspace_bytes(int64_t n_rows) {
  if (n_rows < 0) n_rows = 0;
  return (size_t)(16 + ((n_rows * 4 + 15) / 16) * 16);
}

int ts_kd_fwd_bwd(const void* s, const void* t, const uint8_t* row_mask, int64_t n_rows, int64_t V,
                  int64_t ld_s, int64_t ld_t, float inv_T, float loss_scale, void* workspace,
                  float* loss_out, void* grad, int64_t ld_g, int dtype, ts_stream_t stream) {
  if (!s || !t || !workspace || !loss_out) return TS_ERR_ARG;
  if (n_rows < 0 || V <= 0 || ld_s < V || ld_t < V || (grad && ld_g < V)) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  // one workgroup (or wavefront) per row; mask counts are summed as floats
  if (n_rows > (1 << 24)) return TS_ERR_RANGE;
  const uintptr_t esz = ts::dtype_size(dtype);
  if (((uintptr_t)s | (uintptr_t)t | (uintptr_t)grad) & (esz - 1)) return TS_ERR_ALIGN;
  if ((uintptr_t)workspace & 15u) return TS_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  if (n_rows == 0) {
    // empty batch: sum over nothing divided by zero rows, as the reference does
    hipLaunchKernelGGL(ts::sum_scale_kernel, dim3(1), dim3(1024), 0, st,
                       reinterpret_cast<const float*>(workspace), (int64_t)0, loss_scale,
                       (const int*)nullptr, 0.f, loss_out);
    return ts::check_launch();
  }
  switch (dtype) {
    case TS_F32:
      return ts::launch_kd<float>(s, t, row_mask, n_rows, V, ld_s, ld_t, inv_T, loss_scale,
                                  workspace, loss_out, grad, ld_g, st);
    case TS_BF16:
      return ts::launch_kd<ts::bf16_t>(s, t, row_mask, n_rows, V, ld_s, ld_t, inv_T, loss_scale,
                                       workspace, loss_out, grad, ld_g, st);
    default:
      return ts::launch_kd<ts::f16_t>(s, t, row_mask, n_rows, V, ld_s, ld_t, inv_T, loss_scale,
                                      workspace, loss_out, grad, ld_g, st);
  }
}

int ts_scale_rows(void* grad, int64_t n_rows, int64_t V, int64_t ld_g, const float* g_dev, int dtype,
                  ts_stream_t stream) {
  if (!grad || !g_dev || n_rows < 0 || V < 0 || ld_g < V) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (n_rows == 0 || V == 0) return TS_OK;
  // a contiguous matrix is one long row: keeps gridDim.y within 65535
  if (ld_g == V) {
    V = n_rows * V;
    ld_g = V;
    n_rows = 1;
  }
  if (n_rows > 65535) return TS_ERR_RANGE;
  const int64_t bx = (V + 2047) / 2048;
  if (bx > 0x7fffffffLL) return TS_ERR_RANGE;
  dim3 grid((unsigned)bx, (unsigned)n_rows);
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case TS_F32:
      hipLaunchKernelGGL((ts::scale_rows_kernel<float>), grid, dim3(256), 0, st, (float*)grad, V, ld_g, g_dev);
      break;
    case TS_BF16:
      hipLaunchKernelGGL((ts::scale_rows_kernel<ts::bf16_t>), grid, dim3(256), 0, st, (ts::bf16_t*)grad, V, ld_g, g_dev);
      break;
    default:
      hipLaunchKernelGGL((ts::scale_rows_kernel<ts::f16_t>), grid, dim3(256), 0, st, (ts::f16_t*)grad, V, ld_g, g_dev);
      break;
  }
  return ts::check_launch();
}

int ts_byol_fwd_bwd(const void* x1, const void* y1, const void* x2, const void* y2, int64_t n,
                    int64_t c, float* workspace, float* loss_out, void* gx1, void* gx2, int dtype,
                    ts_stream_t stream) {
  if (!x1 || !y1 || !workspace || !loss_out) return TS_ERR_ARG;
  if ((x2 == nullptr) != (y2 == nullptr)) return TS_ERR_ARG;
  if (n < 0 || c <= 0) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (n > (1 << 28)) return TS_ERR_RANGE;
  hipStream_t st = (hipStream_t)stream;
  if (n == 0) {
    // mean over zero rows: 0/0 = NaN, like torch's mean of an empty tensor
    hipLaunchKernelGGL(ts::sum_scale_kernel, dim3(1), dim3(1024), 0, st, (const float*)workspace,
                       (int64_t)0, 1.0f, (const int*)nullptr, 0.f, loss_out);
    return ts::check_launch();
  }
  switch (dtype) {
    case TS_F32:
      return ts::launch_byol<float>(x1, y1, x2, y2, n, c, workspace, loss_out, gx1, gx2, st);
    case TS_BF16:
      return ts::launch_byol<ts::bf16_t>(x1, y1, x2, y2, n, c, workspace, loss_out, gx1, gx2, st);
    default:
      return ts::launch_byol<ts::f16_t>(x1, y1, x2, y2, n, c, workspace, loss_out, gx1, gx2, st);
  }
}

}  // extern "C"
