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

// ---------------------------------------------------------------------------
// Small planes (HW <= kBnFlatMaxHW): flat tiles.  A plane of a late ResNet
// stage is 49 or 16 elements; a wavefront per plane leaves most lanes idle
// there (and a [N, C, 1, 1] input one lane in 64).  But the C planes of one
// sample are contiguous, so a workgroup takes a range of kBnFlatElems
// consecutive floats of every sample of its slab -- whole 16-byte vectors,
// one per thread and sample, fully coalesced, no index arithmetic in the loop --
// whatever channels that range covers.  A thread's four elements keep the same
// channels from sample to sample, so it accumulates per element in registers;
// at the end the per-position partial sums go through LDS, a thread (planes of
// up to 16 elements) or a wavefront per channel adds up that channel's
// positions, and one atomic add per channel and quantity leaves the workgroup,
// as in the kernels above.  Needs C * HW to be a multiple of 4 and the tensors
// on 16-byte boundaries; everything else keeps the plane kernels.
// Through the C ABI, us: [256, 512, 7, 7] training forward 134 -> 20 and backward
// 160 -> 26; [256, 2048, 7, 7] 316 -> 55-61; [512, 512, 4, 4] 122 -> 14;
// [4096, 512, 1, 1] 794 -> 30.
// ---------------------------------------------------------------------------
constexpr int kBnFlatElems = kBnBlock * 4;
constexpr int64_t kBnFlatMaxHW = 256;
constexpr int kBnFlatMaxCh = kBnFlatElems + 1;  // channels a tile can touch (HW = 1, plus one cut at the front)
constexpr int kBnFlatShiftN = 16;
constexpr int kBnFlatInFlight = 16;  // samples a thread has in flight (one 16-byte vector each); half per operand with two
#ifndef TS_BN_FLAT_SLABS
#define TS_BN_FLAT_SLABS 16
#endif
constexpr int64_t kBnFlatMaxSlabs = TS_BN_FLAT_SLABS;

struct FlatTile {
  uint32_t f0;     // first float of the tile inside a sample
  int nelem;       // floats of the tile (a multiple of 4)
  uint32_t c_lo;   // first channel the tile touches
  int nch;         // channels it touches
  bool valid;      // this thread's vector lies inside the tile
  int ch[4];       // tile-local channel of each of the thread's four elements
};

__device__ __forceinline__ FlatTile flat_tile(int64_t C, int64_t HW) {
  FlatTile t;
  const uint32_t E = (uint32_t)(C * HW), hw = (uint32_t)HW;
  t.f0 = blockIdx.x * (uint32_t)kBnFlatElems;
  t.nelem = (int)((E - t.f0 < (uint32_t)kBnFlatElems) ? E - t.f0 : (uint32_t)kBnFlatElems);
  t.c_lo = t.f0 / hw;
  t.nch = (int)((t.f0 + (uint32_t)t.nelem - 1) / hw - t.c_lo) + 1;
  const int e0 = 4 * (int)threadIdx.x;
  t.valid = e0 < t.nelem;
#pragma unroll
  for (int j = 0; j < 4; ++j) t.ch[j] = t.valid ? (int)((t.f0 + (uint32_t)(e0 + j)) / hw - t.c_lo) : 0;
  return t;
}

// The shift of a channel on this path: the mean of its first (up to) 16
// values in (sample, position) order, added up serially -- the same loads and
// the same order wherever it is computed, so the statistics and the
// normalising launch agree on it to the bit.
__device__ __forceinline__ float flat_shift(const float* __restrict__ x, uint32_t c, int64_t N, int64_t C,
                                            int64_t HW) {
  const int64_t avail = N * HW;
  const int m = avail < kBnFlatShiftN ? (int)avail : kBnFlatShiftN;
  float v[kBnFlatShiftN];
  int64_t n = 0, i = 0;
#pragma unroll
  for (int j = 0; j < kBnFlatShiftN; ++j) {
    v[j] = j < m ? x[(n * C + c) * HW + i] : 0.f;
    if (++i == HW) {
      i = 0;
      ++n;
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < kBnFlatShiftN; ++j) s += v[j];
  return s / (float)m;
}

// Adds up, per channel of the tile, the per-position partial sums in la / lb
// (kBnFlatElems floats each, zeros beyond the tile) and hands (channel, a, b)
// to emit on one thread per channel.
template <typename F>
__device__ __forceinline__ void flat_reduce_channels(const FlatTile& t, int64_t HW, const float* la, const float* lb,
                                                     F emit) {
  const uint32_t hw = (uint32_t)HW;
  auto range = [&](int lc, int& lo, int& hi) {
    const uint32_t c = t.c_lo + (uint32_t)lc;
    const uint32_t b = c * hw, e = b + hw, end = t.f0 + (uint32_t)t.nelem;
    lo = (int)((b > t.f0 ? b : t.f0) - t.f0);
    hi = (int)((e < end ? e : end) - t.f0);
  };
  if (HW <= 16) {
    for (int lc = threadIdx.x; lc < t.nch; lc += kBnBlock) {
      int lo, hi;
      range(lc, lo, hi);
      float a = 0.f, b = 0.f;
      for (int i = lo; i < hi; ++i) {
        a += la[i];
        b += lb[i];
      }
      emit(t.c_lo + (uint32_t)lc, a, b);
    }
  } else {
    const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
    for (int lc = w; lc < t.nch; lc += kBnBlock / kWave) {
      int lo, hi;
      range(lc, lo, hi);
      float a = 0.f, b = 0.f;
      for (int i = lo + lane; i < hi; i += kWave) {
        a += la[i];
        b += lb[i];
      }
      a = wave_sum(a);
      b = wave_sum(b);
      if (lane == 0) emit(t.c_lo + (uint32_t)lc, a, b);
    }
  }
}

// First launch of the fused training forward on small planes: sum(x - k) and
// sum((x - k)^2) per channel into ws.  gridDim = (tiles of a sample, slabs).
__global__ __launch_bounds__(kBnBlock) void bn_flat_stats_kernel(const float* __restrict__ x, int64_t N, int64_t C,
                                                                 int64_t HW, int64_t slab, float* __restrict__ ws) {
  __shared__ float lk[kBnFlatMaxCh];
  __shared__ float ls[kBnFlatElems], lq[kBnFlatElems];
  const FlatTile t = flat_tile(C, HW);
  const int64_t n0 = (int64_t)blockIdx.y * slab;
  const int64_t n1 = (n0 + slab < N) ? n0 + slab : N;
  const int64_t stride4 = C * HW / 4;  // 16-byte vectors per sample
  const f32x4* p = reinterpret_cast<const f32x4*>(x + t.f0) + threadIdx.x;
  // A workgroup's lifetime is a chain of memory round trips (every workgroup of the launch is resident
  // at once), so the first round of loads is on its way before the shifts are worked out, and a round
  // is up to 16 samples.
  constexpr int U = kBnFlatInFlight;
  f32x4 v[U];
  if (t.valid) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (n0 + u < n1) v[u] = p[(n0 + u) * stride4];  // plain loads: the normalising launch reads x again
  }
  for (int lc = threadIdx.x; lc < t.nch; lc += kBnBlock) lk[lc] = flat_shift(x, t.c_lo + (uint32_t)lc, N, C, HW);
  __syncthreads();
  float k[4], S[4] = {0.f, 0.f, 0.f, 0.f}, Q[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 4; ++j) k[j] = lk[t.ch[j]];
  if (t.valid) {
    for (int64_t n = n0; n < n1; n += U) {
      if (n != n0) {
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (n + u < n1) v[u] = p[(n + u) * stride4];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (n + u < n1) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float d = v[u][j] - k[j];
            S[j] += d;
            Q[j] += d * d;
          }
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    ls[4 * threadIdx.x + j] = S[j];
    lq[4 * threadIdx.x + j] = Q[j];
  }
  __syncthreads();
  flat_reduce_channels(t, HW, ls, lq, [&](uint32_t c, float a, float b) {
    unsafeAtomicAdd(ws + c, a);
    unsafeAtomicAdd(ws + C + c, b);
  });
}

// Stand-alone statistics pass on small planes, second launch: one thread per
// channel does what the last workgroup of a channel does in bn_stats_kernel
// (the channel's bookkeeping from the two sums), and clears the sums again.
__global__ __launch_bounds__(kBnBlock) void bn_flat_stats_finish_kernel(const float* __restrict__ x, int64_t N,
                                                                        int64_t C, int64_t HW, float cnt,
                                                                        float* __restrict__ ws, float* sum,
                                                                        float* sum_squares, float* ub_mean,
                                                                        float* ub_invstd, float eps) {
  const int64_t c = (int64_t)blockIdx.x * kBnBlock + threadIdx.x;
  if (c >= C) return;
  const float k = flat_shift(x, (uint32_t)c, N, C, HW);
  const float St = ws[c], Qt = ws[C + c];
  ws[c] = 0.f;
  ws[C + c] = 0.f;
  if (sum) sum[c] += fmaf(cnt, k, St);
  if (sum_squares) sum_squares[c] += fmaf(k, fmaf(cnt, k, 2.f * St), Qt);
  const float dm = St / cnt;  // mean - k
  if (ub_mean) ub_mean[c] = k + dm;
  if (ub_invstd) ub_invstd[c] = 1.f / sqrtf(fmaxf(Qt / cnt - dm * dm, 0.f) + eps);
}

// y = (x - mu) * a + b with per-element constants; MODE 0: fixed statistics
// (mean, invstd or var), MODE 1: second launch of the fused training forward
// (statistics from ws_in; the channel's bookkeeping is done by the workgroup
// of the first slab whose tile holds the channel's first element).
template <int MODE>
__global__ __launch_bounds__(kBnBlock) void bn_flat_apply_kernel(
    const float* __restrict__ x, float* __restrict__ y, const float* __restrict__ mean,
    const float* __restrict__ invstd_or_var, const float* __restrict__ gamma, const float* __restrict__ beta,
    int64_t N, int64_t C, int64_t HW, int64_t slab, int is_var, float cnt, float eps, const float* __restrict__ ws_in,
    float* __restrict__ ws_clear, float* sum, float* sum_squares, float* ub_mean, float* ub_invstd) {
  __shared__ float l_mu[kBnFlatMaxCh], l_a[kBnFlatMaxCh], l_b[kBnFlatMaxCh];
  const FlatTile t = flat_tile(C, HW);
  for (int lc = threadIdx.x; lc < t.nch; lc += kBnBlock) {
    const uint32_t c = t.c_lo + (uint32_t)lc;
    float mu, istd;
    if (MODE == 0) {
      mu = mean[c];
      istd = is_var ? 1.f / sqrtf(invstd_or_var[c] + eps) : invstd_or_var[c];
    } else {
      const float k = flat_shift(x, c, N, C, HW);  // the statistics launch took its sums about the same value
      const float S = ws_in[c], Q = ws_in[C + c];
      const float dm = S / cnt;  // mean - k
      mu = k + dm;
      istd = 1.f / sqrtf(fmaxf(Q / cnt - dm * dm, 0.f) + eps);
      if (blockIdx.y == 0 && c * (uint32_t)HW >= t.f0) {
        if (sum) sum[c] += fmaf(cnt, k, S);
        if (sum_squares) sum_squares[c] += fmaf(k, fmaf(cnt, k, 2.f * S), Q);
        if (ub_mean) ub_mean[c] = mu;
        if (ub_invstd) ub_invstd[c] = istd;
        ws_clear[c] = 0.f;
        ws_clear[C + c] = 0.f;
      }
    }
    l_mu[lc] = mu;
    l_a[lc] = gamma ? istd * gamma[c] : istd;
    l_b[lc] = beta ? beta[c] : 0.f;
  }
  __syncthreads();
  if (!t.valid) return;
  float mu[4], a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    mu[j] = l_mu[t.ch[j]];
    a[j] = l_a[t.ch[j]];
    b[j] = l_b[t.ch[j]];
  }
  const int64_t n0 = (int64_t)blockIdx.y * slab;
  const int64_t n1 = (n0 + slab < N) ? n0 + slab : N;
  const int64_t stride4 = C * HW / 4;
  const f32x4* p = reinterpret_cast<const f32x4*>(x + t.f0) + threadIdx.x;
  f32x4* o = reinterpret_cast<f32x4*>(y + t.f0) + threadIdx.x;
  constexpr int U = kBnFlatInFlight;
  for (int64_t n = n0; n < n1; n += U) {
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (n + u < n1) v[u] = __builtin_nontemporal_load(p + (n + u) * stride4);  // last reader of x in this call
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (n + u < n1) {
        f32x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = (v[u][j] - mu[j]) * a[j] + b[j];
        __builtin_nontemporal_store(r, o + (n + u) * stride4);
      }
    }
  }
}

// Backward on small planes, level 1: per-channel sum(dy) and sum(dy * xhat) into ws.
__global__ __launch_bounds__(kBnBlock) void bn_flat_bwd_reduce_kernel(const float* __restrict__ x,
                                                                      const float* __restrict__ dy,
                                                                      const float* __restrict__ mean,
                                                                      const float* __restrict__ invstd, int64_t N,
                                                                      int64_t C, int64_t HW, int64_t slab,
                                                                      float* __restrict__ ws) {
  __shared__ float l_mu[kBnFlatMaxCh], l_is[kBnFlatMaxCh];
  __shared__ float ls[kBnFlatElems], lq[kBnFlatElems];
  const FlatTile t = flat_tile(C, HW);
  for (int lc = threadIdx.x; lc < t.nch; lc += kBnBlock) {
    l_mu[lc] = mean[t.c_lo + (uint32_t)lc];
    l_is[lc] = invstd[t.c_lo + (uint32_t)lc];
  }
  __syncthreads();
  float mu[4], is[4], A[4] = {0.f, 0.f, 0.f, 0.f}, B[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    mu[j] = l_mu[t.ch[j]];
    is[j] = l_is[t.ch[j]];
  }
  const int64_t n0 = (int64_t)blockIdx.y * slab;
  const int64_t n1 = (n0 + slab < N) ? n0 + slab : N;
  const int64_t stride4 = C * HW / 4;
  const f32x4* px = reinterpret_cast<const f32x4*>(x + t.f0) + threadIdx.x;
  const f32x4* pg = reinterpret_cast<const f32x4*>(dy + t.f0) + threadIdx.x;
  constexpr int U = kBnFlatInFlight / 2;
  if (t.valid) {
    for (int64_t n = n0; n < n1; n += U) {
      f32x4 v[U], g[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (n + u < n1) {
          v[u] = px[(n + u) * stride4];  // plain loads: the dx launch reads both again
          g[u] = pg[(n + u) * stride4];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (n + u < n1) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            A[j] += g[u][j];
            B[j] += g[u][j] * ((v[u][j] - mu[j]) * is[j]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    ls[4 * threadIdx.x + j] = A[j];
    lq[4 * threadIdx.x + j] = B[j];
  }
  __syncthreads();
  flat_reduce_channels(t, HW, ls, lq, [&](uint32_t c, float a, float b) {
    unsafeAtomicAdd(ws + c, a);
    unsafeAtomicAdd(ws + C + c, b);
  });
}

// Backward on small planes, level 2: dx, and dbeta / dgamma / the clearing of
// the other workspace half by the owner of each channel (as in the forward).
__global__ __launch_bounds__(kBnBlock) void bn_flat_bwd_dx_kernel(
    const float* __restrict__ x, const float* __restrict__ dy, const float* __restrict__ mean,
    const float* __restrict__ invstd, const float* __restrict__ gamma, const float* __restrict__ ws_sums,
    float* __restrict__ ws_clear, float* __restrict__ dgamma, float* __restrict__ dbeta, float* __restrict__ dx,
    int64_t N, int64_t C, int64_t HW, int64_t slab, float inv_cnt /* 0: fixed statistics */) {
  __shared__ float l_mu[kBnFlatMaxCh], l_is[kBnFlatMaxCh], l_gi[kBnFlatMaxCh], l_mb[kBnFlatMaxCh], l_mg[kBnFlatMaxCh];
  const FlatTile t = flat_tile(C, HW);
  for (int lc = threadIdx.x; lc < t.nch; lc += kBnBlock) {
    const uint32_t c = t.c_lo + (uint32_t)lc;
    const float istd = invstd[c];
    const float sum_dy = ws_sums[c], sum_dyx = ws_sums[C + c];
    if (blockIdx.y == 0 && c * (uint32_t)HW >= t.f0) {
      dbeta[c] = sum_dy;
      dgamma[c] = sum_dyx;
      ws_clear[c] = 0.f;
      ws_clear[C + c] = 0.f;
    }
    l_mu[lc] = mean[c];
    l_is[lc] = istd;
    l_gi[lc] = (gamma ? gamma[c] : 1.f) * istd;
    l_mb[lc] = sum_dy * inv_cnt;
    l_mg[lc] = sum_dyx * inv_cnt;
  }
  __syncthreads();
  if (!t.valid) return;
  float mu[4], is[4], gi[4], mb[4], mg[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    mu[j] = l_mu[t.ch[j]];
    is[j] = l_is[t.ch[j]];
    gi[j] = l_gi[t.ch[j]];
    mb[j] = l_mb[t.ch[j]];
    mg[j] = l_mg[t.ch[j]];
  }
  const int64_t n0 = (int64_t)blockIdx.y * slab;
  const int64_t n1 = (n0 + slab < N) ? n0 + slab : N;
  const int64_t stride4 = C * HW / 4;
  const f32x4* px = reinterpret_cast<const f32x4*>(x + t.f0) + threadIdx.x;
  const f32x4* pg = reinterpret_cast<const f32x4*>(dy + t.f0) + threadIdx.x;
  f32x4* pd = reinterpret_cast<f32x4*>(dx + t.f0) + threadIdx.x;
  constexpr int U = kBnFlatInFlight / 2;
  for (int64_t n = n0; n < n1; n += U) {
    f32x4 v[U], g[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (n + u < n1) {
        v[u] = __builtin_nontemporal_load(px + (n + u) * stride4);  // second and last pass over x and dy
        g[u] = __builtin_nontemporal_load(pg + (n + u) * stride4);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (n + u < n1) {
        f32x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = gi[j] * (g[u][j] - mb[j] - ((v[u][j] - mu[j]) * is[j]) * mg[j]);
        __builtin_nontemporal_store(r, pd + (n + u) * stride4);
      }
    }
  }
}

// Whether a call takes the flat kernels, and how many samples a workgroup gets.
inline bool bn_flat_ok(int64_t C, int64_t HW, uintptr_t ptr_bits) {
  return HW <= kBnFlatMaxHW && (C * HW) % 4 == 0 && (ptr_bits & 15u) == 0;
}

inline void bn_flat_grid(int64_t N, int64_t C, int64_t HW, dim3* grid, int64_t* slab) {
  const int64_t tiles = (C * HW + kBnFlatElems - 1) / kBnFlatElems;
  // About 1024 workgroups, but at most kBnFlatMaxSlabs slabs: every slab's workgroup sends one atomic
  // add per channel and quantity to the same few addresses, and those are served one after the other
  // (64 slabs on [256, 512, 7, 7]: 36 us for the statistics, most of it that queue).
  int64_t slabs = (1024 + tiles - 1) / tiles;
  // (with only a few tiles the slabs are all the parallelism there is: twice the cap)
  const int64_t cap = tiles >= 16 ? kBnFlatMaxSlabs : 2 * kBnFlatMaxSlabs;
  if (slabs > cap) slabs = cap;
  if (slabs > (N + 3) / 4) slabs = (N + 3) / 4;
  if (slabs < 1) slabs = 1;
  const int64_t per = (N + slabs - 1) / slabs;
  *slab = per;
  *grid = dim3((unsigned)tiles, (unsigned)((N + per - 1) / per));
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
  if (ts::bn_flat_ok(C, HW, (uintptr_t)x)) {
    // small planes: the flat-tile sums, then a launch of one thread per channel (two short launches
    // instead of the one below, which would leave most of its lanes idle on such planes)
    dim3 fgrid;
    int64_t fslab;
    ts::bn_flat_grid(N, C, HW, &fgrid, &fslab);
    hipLaunchKernelGGL(ts::bn_flat_stats_kernel, fgrid, dim3(ts::kBnBlock), 0, st, x, N, C, HW, fslab, ws);
    rc = ts::check_launch();
    if (rc) return rc;
    hipLaunchKernelGGL(ts::bn_flat_stats_finish_kernel, dim3((unsigned)((C + ts::kBnBlock - 1) / ts::kBnBlock)),
                       dim3(ts::kBnBlock), 0, st, x, N, C, HW, cnt, ws, sum, sum_squares, ub_mean, ub_invstd, eps);
    return ts::check_launch();
  }
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
  if (ts::bn_flat_ok(C, HW, (uintptr_t)x | (uintptr_t)y)) {
    dim3 fgrid;
    int64_t fslab;
    ts::bn_flat_grid(N, C, HW, &fgrid, &fslab);
    hipLaunchKernelGGL(ts::bn_flat_apply_kernel<0>, fgrid, dim3(ts::kBnBlock), 0, (hipStream_t)stream, x, y, mean,
                       invstd_or_var, gamma, beta, N, C, HW, fslab, is_var, 0.f, eps, (const float*)nullptr,
                       (float*)nullptr, (float*)nullptr, (float*)nullptr, (float*)nullptr, (float*)nullptr);
    return ts::check_launch();
  }
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
  if (ts::bn_flat_ok(C, HW, (uintptr_t)x | (uintptr_t)y)) {
    dim3 fgrid;
    int64_t fslab;
    ts::bn_flat_grid(N, C, HW, &fgrid, &fslab);
    hipLaunchKernelGGL(ts::bn_flat_stats_kernel, fgrid, dim3(ts::kBnBlock), 0, st, x, N, C, HW, fslab, ws_now);
    rc = ts::check_launch();
    if (rc) return rc;
    hipLaunchKernelGGL(ts::bn_flat_apply_kernel<1>, fgrid, dim3(ts::kBnBlock), 0, st, x, y, (const float*)nullptr,
                       (const float*)nullptr, gamma, beta, N, C, HW, fslab, 0, (float)((double)N * (double)HW), eps,
                       (const float*)ws_now, ws_other, sum, sum_squares, ub_mean, ub_invstd);
    return ts::check_launch();
  }
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
  if (ts::bn_flat_ok(C, HW, (uintptr_t)x | (uintptr_t)dy | (uintptr_t)dx)) {
    dim3 fgrid;
    int64_t fslab;
    ts::bn_flat_grid(N, C, HW, &fgrid, &fslab);
    hipLaunchKernelGGL(ts::bn_flat_bwd_reduce_kernel, fgrid, dim3(ts::kBnBlock), 0, st, x, dy, ub_mean, ub_invstd, N, C,
                       HW, fslab, ws_now);
    rc = ts::check_launch();
    if (rc) return rc;
    hipLaunchKernelGGL(ts::bn_flat_bwd_dx_kernel, fgrid, dim3(ts::kBnBlock), 0, st, x, dy, ub_mean, ub_invstd, gamma,
                       (const float*)ws_now, ws_other, dgamma, dbeta, dx, N, C, HW, fslab,
                       training ? (float)(1.0 / ((double)N * (double)HW)) : 0.f);
    return ts::check_launch();
  }
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
