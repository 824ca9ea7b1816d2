// DeferredBatchNorm kernels for fp32 [N, C, HW] activations.
//
// Work decomposition shared by every per-element kernel here: a workgroup
// owns one channel c and a slab of consecutive samples n0..n1; inside a
// sample the channel's HW values are contiguous, so the accesses are 16-byte
// vectors over runs of HW floats.  gridDim = (slabs, C).
//
// Reductions are two-level: registers -> LDS tree inside the workgroup, then
// one hardware fp32 atomic add per workgroup and quantity into a small float
// workspace.  The workspace is zero between calls: whoever consumes it (the
// last workgroup of a channel in the stand-alone statistics pass, the
// normalising kernel in the fused passes) also clears it.
//
// Sums are taken about a per-channel shift k_c (the mean of the channel's
// first 64 values, bn_shift): S' = sum(x - k), Q' = sum((x - k)^2).  The
// variance Q'/n - (S'/n)^2 then cancels against (mean - k)^2, which is far
// below the variance itself, instead of against mean^2; the raw sums the
// reference accumulates follow exactly as  sum x = S' + n k  and
// sum x^2 = Q' + 2 k S' + n k^2.
#include "common.h"

namespace ts {

constexpr int kBnBlock = 256;
constexpr int kBnUnroll = 4;

// The per-channel shift the sums are taken about: the mean of the first (up
// to) 64 values of the channel's first plane.  Every wavefront of every
// workgroup of the channel computes it from the same loads in the same order,
// so all agree to the bit.  A single sample as the shift can sit several
// standard deviations from the mean, and (mean - k)^2, which the sums then
// carry and the reconstruction takes out again, costs a digit of the
// accumulated sum of squares; the mean of 64 samples is within sigma / 8.
__device__ __forceinline__ float bn_shift(const float* __restrict__ x, int64_t c, int64_t HW) {
  const int lane = threadIdx.x % kWave;
  const int m = HW < kWave ? (int)HW : kWave;
  const float v = lane < m ? x[c * HW + lane] : 0.f;
  return wave_sum(v) / (float)m;
}

struct PlaneSplit {
  int64_t head, nvec, tail0;  // scalar head, 16-byte vectors, first tail element
};

__device__ __forceinline__ PlaneSplit split_plane(const float* p, int64_t HW) {
  PlaneSplit s;
  s.head = (int64_t)(((16u - (uint32_t)((uintptr_t)p & 15u)) & 15u) >> 2);
  if (s.head > HW) s.head = HW;
  s.nvec = (HW - s.head) >> 2;
  s.tail0 = s.head + (s.nvec << 2);
  return s;
}

// Accumulates (a, b) over the slab's elements of x (and optionally a second
// tensor y with the same layout) through a functor: f(xv, yv, a, b), with a
// wavefront per plane: wavefront w of the workgroup takes planes n0 + w,
// n0 + w + NW, ...  A plane of a small feature map is a few hundred 16-byte
// vectors; dealt to 64 lanes instead of a whole workgroup, nearly every load
// instruction has all its lanes at work (a 56 x 56 plane is 784 vectors: 12.25
// per lane, against 3.06 per thread of a 256-thread workgroup, whose fourth
// load has 16 threads in it).  Four loads per lane and operand are in flight at
// a time; more of them (8, 14: the whole plane) were measured slower.
constexpr int kBnWaveLoads = 4;   // 16-byte loads per lane in flight, one operand (2 and 3: 1-2 % slower)
constexpr int kBnWaveLoads2 = 2;  // per operand when there are two (backward 80.3 us against 83.2 with 4; 1: 80.1, 6: 82.6)
// STREAM: the operands are not read again by a kernel of the same call, so
// they are fetched with non-temporal loads (the stand-alone statistics pass:
// 20.4 against 22.2 us on 103 MB; the statistics half of the fused forward
// leaves its input to the normalising half with plain loads, which otherwise
// takes 10 us longer).
template <bool TWO, bool STREAM, int BLOCK = kBnBlock, typename F>
__device__ __forceinline__ void slab_reduce_waves(const float* __restrict__ x, const float* __restrict__ y, int64_t n0,
                                                  int64_t n1, int64_t C, int64_t c, int64_t HW, float& a, float& b,
                                                  F f) {
  constexpr int NW = BLOCK / kWave;
  constexpr int U = TWO ? kBnWaveLoads2 : kBnWaveLoads;
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  for (int64_t n = n0 + w; n < n1; n += NW) {
    const int64_t off = (n * C + c) * HW;
    const float* px = x + off;
    const float* py = TWO ? y + off : nullptr;
    const PlaneSplit sp = split_plane(px, HW);
    const bool yvec = !TWO || ((((uintptr_t)py) & 15u) == (((uintptr_t)px) & 15u));
    const f32x4* px4 = reinterpret_cast<const f32x4*>(px + sp.head);
    const f32x4* py4 = reinterpret_cast<const f32x4*>(py + sp.head);
    for (int64_t base = 0; base < sp.nvec; base += kWave * U) {
      f32x4 v[U], vy[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = base + u * kWave + lane;
        if (i < sp.nvec) {
          v[u] = STREAM ? __builtin_nontemporal_load(px4 + i) : px4[i];
          if (TWO) {
            if (yvec) {
              vy[u] = STREAM ? __builtin_nontemporal_load(py4 + i) : py4[i];
            } else {
              const float* q = py + sp.head + (i << 2);
              vy[u] = f32x4{q[0], q[1], q[2], q[3]};
            }
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = base + u * kWave + lane;
        if (i < sp.nvec) {
          f(v[u].x, TWO ? vy[u].x : 0.f, a, b);
          f(v[u].y, TWO ? vy[u].y : 0.f, a, b);
          f(v[u].z, TWO ? vy[u].z : 0.f, a, b);
          f(v[u].w, TWO ? vy[u].w : 0.f, a, b);
        }
      }
    }
    if (lane < sp.head) f(px[lane], TWO ? py[lane] : 0.f, a, b);
    const int64_t it = sp.tail0 + lane;
    if (it < HW) f(px[it], TWO ? py[it] : 0.f, a, b);
  }
}

// Statistics of one micro-batch in ONE launch: every workgroup adds its slab's
// sums into the workspace with returning atomics, then takes a ticket from the
// channel's counter; the workgroup that draws the last ticket knows that all
// other additions have been performed (each was complete before its ticket
// was drawn), collects the totals with atomic exchanges -- which also leave
// the workspace zero for the next call -- and does the channel's bookkeeping.
// Atomics act at the device's point of coherence, so no cache has to be
// flushed or invalidated for this hand-off.
//   ws: [0, C) sum(x - k), [C, 2C) sum((x - k)^2), [2C, 3C) tickets (as uint32)
// FINAL = false is the first launch of the fused passes: sums only, the
// launch that follows consumes them.
template <bool FINAL>
__global__ __launch_bounds__(kBnBlock) void bn_stats_kernel(const float* __restrict__ x, int64_t N,
                                                            int64_t C, int64_t HW, int64_t slab, float cnt,
                                                            float* __restrict__ ws, float* sum,
                                                            float* sum_squares, float* ub_mean,
                                                            float* ub_invstd, float eps) {
  __shared__ float lds[kBnBlock / kWave];
  const int64_t c = blockIdx.y;
  const int64_t n0 = (int64_t)blockIdx.x * slab;
  const int64_t n1 = (n0 + slab < N) ? n0 + slab : N;
  const float k = bn_shift(x, c, HW);
  float S = 0.f, Q = 0.f;
  slab_reduce_waves<false, FINAL>(x, nullptr, n0, n1, C, c, HW, S, Q, [k](float xv, float, float& a, float& b) {
    const float d = xv - k;
    a += d;
    b += d * d;
  });
  S = block_sum<kBnBlock / kWave>(S, lds);
  Q = block_sum<kBnBlock / kWave>(Q, lds);
  if (!FINAL) {
    if (threadIdx.x == 0) {
      unsafeAtomicAdd(ws + c, S);
      unsafeAtomicAdd(ws + C + c, Q);
    }
    return;
  }
  if (threadIdx.x == 0) {
    unsigned* tickets = reinterpret_cast<unsigned*>(ws + 2 * C);
    // the returned values are waited for: the additions are done before the ticket is drawn
    const float r0 = atomicAdd(ws + c, S);
    const float r1 = atomicAdd(ws + C + c, Q);
    asm volatile("" ::"v"(r0), "v"(r1) : "memory");
    const unsigned ticket = atomicAdd(tickets + c, 1u);
    if (ticket == gridDim.x - 1) {
      const float St = atomicExch(ws + c, 0.f), Qt = atomicExch(ws + C + c, 0.f);
      atomicExch(tickets + c, 0u);
      // sum x = S' + n k and sum x^2 = Q' + k (2 S' + n k), each with one rounding per step
      if (sum) sum[c] += fmaf(cnt, k, St);
      if (sum_squares) sum_squares[c] += fmaf(k, fmaf(cnt, k, 2.f * St), Qt);
      const float dm = St / cnt;  // mean - k
      if (ub_mean) ub_mean[c] = k + dm;
      if (ub_invstd) ub_invstd[c] = 1.f / sqrtf(fmaxf(Qt / cnt - dm * dm, 0.f) + eps);
    }
  }
}

// The reference's rounding order, one fp32 operation at a time:
//   mean = sum / counter;  var = sum_squares / counter - mean**2
//   running *= (1 - f);  running += stat * f
// One workgroup walks all channels (a few thousand at most), so that the
// counter can be read by every thread, then bumped, inside one launch.
constexpr int kBnCommitBlock = 1024;
__global__ __launch_bounds__(kBnCommitBlock) void bn_commit_kernel(float* __restrict__ sum,
                                                                   float* __restrict__ sum_squares,
                                                                   float* __restrict__ running_mean,
                                                                   float* __restrict__ running_var,
                                                                   int64_t* __restrict__ nbt, int64_t C, float counter,
                                                                   double momentum) {
  // the value used is "after the increment"; thread 0 stores it once every thread has read the old one
  const int64_t tracked = nbt ? *nbt + 1 : 1;
  __syncthreads();
  if (nbt && threadIdx.x == 0) *nbt = tracked;
  const double f = (momentum < 0.0) ? 1.0 / (double)tracked : momentum;
  const float f32 = (float)f, omf32 = (float)(1.0 - f);
  for (int64_t c = threadIdx.x; c < C; c += kBnCommitBlock) {
#pragma clang fp contract(off)
    const float mean = sum[c] / counter;
    const float msq = mean * mean;
    const float var = sum_squares[c] / counter - msq;
    const float rm = running_mean[c] * omf32, dm = mean * f32;
    const float rv = running_var[c] * omf32, dv = var * f32;
    running_mean[c] = rm + dm;
    running_var[c] = rv + dv;
    sum[c] = 0.f;
    sum_squares[c] = 0.f;
  }
}

// y = (x - mu) * a + b over this workgroup's slab of channel c
__device__ __forceinline__ void bn_apply_slab(const float* __restrict__ x, float* __restrict__ y, int64_t N,
                                              int64_t C, int64_t HW, int64_t slab, int64_t c, float mu, float a,
                                              float b) {
  const int64_t n0 = (int64_t)blockIdx.x * slab;
  const int64_t n1 = (n0 + slab < N) ? n0 + slab : N;
  // a wavefront per plane, as in slab_reduce_waves
  constexpr int kStep = kWave;
  const int tid = threadIdx.x % kWave;
  const int64_t nfirst = n0 + threadIdx.x / kWave, nstep = kBnBlock / kWave;
  for (int64_t n = nfirst; n < n1; n += nstep) {
    const int64_t off = (n * C + c) * HW;
    const float* px = x + off;
    float* py = y + off;
    const PlaneSplit sp = split_plane(px, HW);
    const bool yvec = (((uintptr_t)py) & 15u) == (((uintptr_t)px) & 15u);
    if (tid < sp.head) py[tid] = (px[tid] - mu) * a + b;
    const f32x4* px4 = reinterpret_cast<const f32x4*>(px + sp.head);
    f32x4* py4 = reinterpret_cast<f32x4*>(py + sp.head);
    for (int64_t base = 0; base < sp.nvec; base += kStep * kBnUnroll) {
      f32x4 v[kBnUnroll];
#pragma unroll
      for (int u = 0; u < kBnUnroll; ++u) {
        const int64_t i = base + u * kStep + tid;
        if (i < sp.nvec) v[u] = __builtin_nontemporal_load(px4 + i);  // last reader of x in this call
      }
#pragma unroll
      for (int u = 0; u < kBnUnroll; ++u) {
        const int64_t i = base + u * kStep + tid;
        if (i < sp.nvec) {
          f32x4 r;
          r.x = (v[u].x - mu) * a + b;
          r.y = (v[u].y - mu) * a + b;
          r.z = (v[u].z - mu) * a + b;
          r.w = (v[u].w - mu) * a + b;
          if (yvec) {
            __builtin_nontemporal_store(r, py4 + i);
          } else {
            float* q = py + sp.head + (i << 2);
            q[0] = r.x;
            q[1] = r.y;
            q[2] = r.z;
            q[3] = r.w;
          }
        }
      }
    }
    const int64_t it = sp.tail0 + tid;
    if (it < HW) py[it] = (px[it] - mu) * a + b;
  }
}

__global__ __launch_bounds__(kBnBlock) void bn_apply_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                            const float* __restrict__ mean,
                                                            const float* __restrict__ invstd_or_var,
                                                            const float* __restrict__ gamma,
                                                            const float* __restrict__ beta, int64_t N,
                                                            int64_t C, int64_t HW, int64_t slab, int is_var,
                                                            float eps) {
  const int64_t c = blockIdx.y;
  const float mu = mean[c];
  const float istd = is_var ? 1.f / sqrtf(invstd_or_var[c] + eps) : invstd_or_var[c];
  const float a = gamma ? istd * gamma[c] : istd;
  const float b = beta ? beta[c] : 0.f;
  bn_apply_slab(x, y, N, C, HW, slab, c, mu, a, b);
}

// Training forward, second launch: normalises with the micro-batch statistics
// that bn_stats_kernel left in `ws_in` (every workgroup derives mean and
// 1/std of its channel from the two sums itself), and the first workgroup of
// each channel does the channel's bookkeeping -- running sums,
// saved statistics -- except that it clears the OTHER workspace half: this
// one is still being read by the channel's other workgroups, the other one
// was consumed by the previous call.
__global__ __launch_bounds__(kBnBlock) void bn_apply_train_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                  const float* __restrict__ gamma,
                                                                  const float* __restrict__ beta, int64_t N,
                                                                  int64_t C, int64_t HW, int64_t slab, float cnt,
                                                                  float eps, const float* __restrict__ ws_in,
                                                                  float* __restrict__ ws_clear, float* sum,
                                                                  float* sum_squares, float* ub_mean,
                                                                  float* ub_invstd) {
  const int64_t c = blockIdx.y;
  const float S = ws_in[c], Q = ws_in[C + c];
  const float k = bn_shift(x, c, HW);  // the statistics launch took its sums about the same value
  const float dm = S / cnt;  // mean - k
  const float mu = k + dm;
  const float istd = 1.f / sqrtf(fmaxf(Q / cnt - dm * dm, 0.f) + eps);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (sum) sum[c] += fmaf(cnt, k, S);
    if (sum_squares) sum_squares[c] += fmaf(k, fmaf(cnt, k, 2.f * S), Q);
    if (ub_mean) ub_mean[c] = mu;
    if (ub_invstd) ub_invstd[c] = istd;
    ws_clear[c] = 0.f;
    ws_clear[C + c] = 0.f;
  }
  const float a = gamma ? istd * gamma[c] : istd;
  const float b = beta ? beta[c] : 0.f;
  bn_apply_slab(x, y, N, C, HW, slab, c, mu, a, b);
}

// Backward, level 1: per-channel sum(dy) and sum(dy * xhat) into ws.
__global__ __launch_bounds__(kBnBlock) void bn_bwd_reduce_kernel(const float* __restrict__ x,
                                                                 const float* __restrict__ dy,
                                                                 const float* __restrict__ mean,
                                                                 const float* __restrict__ invstd, int64_t N,
                                                                 int64_t C, int64_t HW, int64_t slab,
                                                                 float* __restrict__ ws) {
  __shared__ float lds[kBnBlock / kWave];
  const int64_t c = blockIdx.y;
  const int64_t n0 = (int64_t)blockIdx.x * slab;
  const int64_t n1 = (n0 + slab < N) ? n0 + slab : N;
  const float mu = mean[c], istd = invstd[c];
  float sdy = 0.f, sdyx = 0.f;
  slab_reduce_waves<true, false>(x, dy, n0, n1, C, c, HW, sdy, sdyx, [mu, istd](float xv, float g, float& a, float& b) {
    a += g;
    b += g * ((xv - mu) * istd);
  });
  sdy = block_sum<kBnBlock / kWave>(sdy, lds);
  sdyx = block_sum<kBnBlock / kWave>(sdyx, lds);
  if (threadIdx.x == 0) {
    unsafeAtomicAdd(ws + c, sdy);
    unsafeAtomicAdd(ws + C + c, sdyx);
  }
}

// Backward, level 2: dx = gamma*invstd*(dy - dbeta/cnt - xhat*dgamma/cnt).
// Every workgroup takes its channel's two sums straight from the reduction
// workspace; the channel's first workgroup also hands them out as dbeta and
// dgamma and, because its siblings are still reading them, clears the OTHER
// of the two alternating workspace halves (the one the previous call used).
__global__ __launch_bounds__(kBnBlock) void bn_bwd_dx_kernel(const float* __restrict__ x,
                                                             const float* __restrict__ dy,
                                                             const float* __restrict__ mean,
                                                             const float* __restrict__ invstd,
                                                             const float* __restrict__ gamma,
                                                             const float* __restrict__ ws_sums,
                                                             float* __restrict__ ws_clear,
                                                             float* __restrict__ dgamma,
                                                             float* __restrict__ dbeta,
                                                             float* __restrict__ dx, int64_t N, int64_t C,
                                                             int64_t HW, int64_t slab, float inv_cnt /* 0: fixed statistics */) {
  const int64_t c = blockIdx.y;
  const int64_t n0 = (int64_t)blockIdx.x * slab;
  const int64_t n1 = (n0 + slab < N) ? n0 + slab : N;
  const float mu = mean[c], istd = invstd[c];
  const float gi = (gamma ? gamma[c] : 1.f) * istd;
  const float sum_dy = ws_sums[c], sum_dyx = ws_sums[C + c];
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    dbeta[c] = sum_dy;
    dgamma[c] = sum_dyx;
    ws_clear[c] = 0.f;
    ws_clear[C + c] = 0.f;
  }
  const float mb = sum_dy * inv_cnt, mg = sum_dyx * inv_cnt;
  // a wavefront per plane, as in slab_reduce_waves
  constexpr int kStep = kWave;
  const int tid = threadIdx.x % kWave;
  auto one = [=](float xv, float g) { return gi * (g - mb - ((xv - mu) * istd) * mg); };
  for (int64_t n = n0 + threadIdx.x / kWave; n < n1; n += kBnBlock / kWave) {
    const int64_t off = (n * C + c) * HW;
    const float* px = x + off;
    const float* pg = dy + off;
    float* pd = dx + off;
    const PlaneSplit sp = split_plane(px, HW);
    const bool vec = ((((uintptr_t)pg) & 15u) == (((uintptr_t)px) & 15u)) &&
                     ((((uintptr_t)pd) & 15u) == (((uintptr_t)px) & 15u));
    if (!vec) {
      for (int64_t i = tid; i < HW; i += kStep) pd[i] = one(px[i], pg[i]);
      continue;
    }
    if (tid < sp.head) pd[tid] = one(px[tid], pg[tid]);
    const f32x4* px4 = reinterpret_cast<const f32x4*>(px + sp.head);
    const f32x4* pg4 = reinterpret_cast<const f32x4*>(pg + sp.head);
    f32x4* pd4 = reinterpret_cast<f32x4*>(pd + sp.head);
    for (int64_t base = 0; base < sp.nvec; base += kStep * kBnUnroll) {
      f32x4 vx[kBnUnroll], vg[kBnUnroll];
#pragma unroll
      for (int u = 0; u < kBnUnroll; ++u) {
        const int64_t i = base + u * kStep + tid;
        if (i < sp.nvec) {
          vx[u] = __builtin_nontemporal_load(px4 + i);  // second and last pass over x and dy
          vg[u] = __builtin_nontemporal_load(pg4 + i);
        }
      }
#pragma unroll
      for (int u = 0; u < kBnUnroll; ++u) {
        const int64_t i = base + u * kStep + tid;
        if (i < sp.nvec) {
          f32x4 r;
          r.x = one(vx[u].x, vg[u].x);
          r.y = one(vx[u].y, vg[u].y);
          r.z = one(vx[u].z, vg[u].z);
          r.w = one(vx[u].w, vg[u].w);
          __builtin_nontemporal_store(r, pd4 + i);
        }
      }
    }
    const int64_t it = sp.tail0 + tid;
    if (it < HW) pd[it] = one(px[it], pg[it]);
  }
}

// Samples per workgroup: about 8K elements each, so small feature maps do
// not degenerate into one workgroup per few hundred bytes.
// Samples per workgroup: about `target` elements.  The fused passes use 8192;
// the stand-alone statistics pass, whose workgroups end with a few dependent
// atomics, is a little faster with twice that (fewer, longer workgroups).
inline int64_t bn_slab(int64_t N, int64_t HW, int64_t target = 8192) {
  int64_t s = (target + HW - 1) / HW;
  constexpr int64_t kw = kBnBlock / kWave;
  s = (s + kw - 1) / kw * kw;  // a wavefront per plane
  if (s < 1) s = 1;
  if (s > N) s = N;
  return s;
}

inline int bn_check_dims(int64_t N, int64_t C, int64_t HW) {
  if (N <= 0 || C <= 0 || HW <= 0) return TS_ERR_ARG;
  if (C > 65535) return TS_ERR_RANGE;  // gridDim.y
  if (N > 0x7fffffffLL) return TS_ERR_RANGE;
  return TS_OK;
}

}  // namespace ts

extern "C" {

size_t ts_bn_stats_workspace_bytes(int64_t C) { return C > 0 ? (size_t)C * 3 * sizeof(float) : 0; }

int ts_bn_stats(const float* x, int64_t N, int64_t C, int64_t HW, float* ws, float* sum,
                float* sum_squares, float* ub_mean, float* ub_invstd, float eps, ts_stream_t stream) {
  if (!x || !ws) return TS_ERR_ARG;
  if ((ub_mean == nullptr) != (ub_invstd == nullptr)) return TS_ERR_ARG;
  if ((sum == nullptr) != (sum_squares == nullptr)) return TS_ERR_ARG;
  int rc = ts::bn_check_dims(N, C, HW);
  if (rc) return rc;
  if ((uintptr_t)x & 3u) return TS_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const float cnt = (float)((double)N * (double)HW);
  const int64_t slab = ts::bn_slab(N, HW, 16384);
  dim3 grid((unsigned)((N + slab - 1) / slab), (unsigned)C);
  hipLaunchKernelGGL(ts::bn_stats_kernel<true>, grid, dim3(ts::kBnBlock), 0, st, x, N, C, HW, slab,
                     cnt, ws, sum, sum_squares, ub_mean, ub_invstd, eps);
  return ts::check_launch();
}

int ts_bn_commit(float* sum, float* sum_squares, float* running_mean, float* running_var,
                 int64_t* num_batches_tracked, int64_t C, double counter, double momentum,
                 ts_stream_t stream) {
  if (!sum || !sum_squares || !running_mean || !running_var) return TS_ERR_ARG;
  if (C <= 0) return TS_ERR_ARG;
  if (momentum < 0.0 && !num_batches_tracked) return TS_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(ts::bn_commit_kernel, dim3(1), dim3(ts::kBnCommitBlock), 0, st, sum, sum_squares, running_mean,
                     running_var, num_batches_tracked, C, (float)counter, momentum);
  return ts::check_launch();
}

int ts_bn_apply(const float* x, float* y, const float* mean, const float* invstd_or_var,
                const float* gamma, const float* beta, int64_t N, int64_t C, int64_t HW, int is_var,
                float eps, ts_stream_t stream) {
  if (!x || !y || !mean || !invstd_or_var) return TS_ERR_ARG;
  int rc = ts::bn_check_dims(N, C, HW);
  if (rc) return rc;
  if (((uintptr_t)x | (uintptr_t)y) & 3u) return TS_ERR_ALIGN;
  const int64_t slab = ts::bn_slab(N, HW);
  dim3 grid((unsigned)((N + slab - 1) / slab), (unsigned)C);
  hipLaunchKernelGGL(ts::bn_apply_kernel, grid, dim3(ts::kBnBlock), 0, (hipStream_t)stream, x, y, mean,
                     invstd_or_var, gamma, beta, N, C, HW, slab, is_var, eps);
  return ts::check_launch();
}

int ts_bn_forward_train(const float* x, float* y, const float* gamma, const float* beta, int64_t N, int64_t C,
                        int64_t HW, float* sum, float* sum_squares, float* ub_mean, float* ub_invstd, float* ws,
                        int parity, float eps, ts_stream_t stream) {
  if (!x || !y || !ws || (parity != 0 && parity != 1)) return TS_ERR_ARG;
  int rc = ts::bn_check_dims(N, C, HW);
  if (rc) return rc;
  if (((uintptr_t)x | (uintptr_t)y) & 3u) return TS_ERR_ALIGN;
  const int64_t slab = ts::bn_slab(N, HW);
  dim3 grid((unsigned)((N + slab - 1) / slab), (unsigned)C);
  hipStream_t st = (hipStream_t)stream;
  float* ws_now = ws + (int64_t)parity * 2 * C;
  float* ws_other = ws + (int64_t)(1 - parity) * 2 * C;
  hipLaunchKernelGGL(ts::bn_stats_kernel<false>, grid, dim3(ts::kBnBlock), 0, st, x, N, C, HW, slab, 0.f, ws_now,
                     (float*)nullptr, (float*)nullptr, (float*)nullptr, (float*)nullptr, 0.f);
  rc = ts::check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(ts::bn_apply_train_kernel, grid, dim3(ts::kBnBlock), 0, st, x, y, gamma, beta, N, C, HW, slab,
                     (float)((double)N * (double)HW), eps, ws_now, ws_other, sum, sum_squares, ub_mean, ub_invstd);
  return ts::check_launch();
}

int ts_bn_backward(const float* x, const float* dy, const float* ub_mean, const float* ub_invstd,
                   const float* gamma, float* dx, float* dgamma, float* dbeta, float* ws, int parity,
                   int64_t N, int64_t C, int64_t HW, int training, ts_stream_t stream) {
  if (!x || !dy || !ub_mean || !ub_invstd || !dx || !dgamma || !dbeta || !ws) return TS_ERR_ARG;
  if (parity != 0 && parity != 1) return TS_ERR_ARG;
  int rc = ts::bn_check_dims(N, C, HW);
  if (rc) return rc;
  if (((uintptr_t)x | (uintptr_t)dy | (uintptr_t)dx) & 3u) return TS_ERR_ALIGN;
  const int64_t slab = ts::bn_slab(N, HW);
  dim3 grid((unsigned)((N + slab - 1) / slab), (unsigned)C);
  hipStream_t st = (hipStream_t)stream;
  float* ws_now = ws + (int64_t)parity * 2 * C;
  float* ws_other = ws + (int64_t)(1 - parity) * 2 * C;
  hipLaunchKernelGGL(ts::bn_bwd_reduce_kernel, grid, dim3(ts::kBnBlock), 0, st, x, dy, ub_mean, ub_invstd,
                     N, C, HW, slab, ws_now);
  rc = ts::check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(ts::bn_bwd_dx_kernel, grid, dim3(ts::kBnBlock), 0, st, x, dy, ub_mean, ub_invstd,
                     gamma, ws_now, ws_other, dgamma, dbeta, dx, N, C, HW, slab,
                     training ? (float)(1.0 / ((double)N * (double)HW)) : 0.f);
  return ts::check_launch();
}

}  // extern "C"
