// MoCo-v3 InfoNCE loss, forward and backward, with every product and sum in
// fp32: the path for fp32 inputs (the reference's TSPipe MoCo run is fp32 end
// to end), for feature widths other than 64 / 128 / 256 (up to 512) and for
// temperatures below the bf16 path's limit.
//
//   qh = q/|q|, kh = k/|k|, logits = qh kh^T / tau,
//   loss = 2 tau * mean_i( lse_i - logits_ii ),
//   dqh_i = (2/N) (sum_j P_ij kh_j - kh_i),  P = softmax(logits) row-wise,
//   dq_i  = (dqh_i - qh_i <qh_i, dqh_i>) / |q_i|.
//
// Same flash-attention shape as the bf16 path (S^T = Kh Q^T, O^T += Kh^T P,
// the N x N logits never stored), on v_mfma_f32_32x32x2_f32, whose products
// and accumulation are fp32.  Differences:
//   * a running row maximum instead of a fixed reference point, so any
//     temperature works; key splits carry their maximum and are merged by the
//     combine kernel;
//   * P is never rounded; the positive key's term is still kept out of O and
//     out of the row sum (l_neg), so that 1 - P_ii/l is formed as l_neg / l
//     without cancellation when P_ii -> 1;
//   * the loss uses the positive logit itself, lse_i - logit_ii
//     = ln2 (m_i + log2 l_i - s_ii), which stays finite when P_ii underflows.
//
// Kernels:
//   norm     one wavefront per row: rq = 1/max(|q|, eps), rk likewise.
//   main     grid (q tile of 128 rows, key split, pair x feature group); 4
//            wavefronts, each owning 32 q rows with their Q fragments in
//            registers.  Keys come in tiles of 32 through LDS (normalised on
//            the way in, fp32, row stride CP+1 words so that both operand
//            reads are free of bank conflicts), two buffers.  A wavefront
//            accumulates O^T for FBW 32-feature blocks; widths above 256
//            are covered by several feature groups, each recomputing S.
//   combine  one wavefront per row: merges the key splits, forms dq, leaves the
//            row's loss term.
//   sum      one workgroup adds up the loss terms in a fixed order.
//
// MFMA 32x32x2 operand layout (lane l, half h = l/32):
//   A: row l%32, contraction slot h;  B: column l%32, slot h;
//   D[i]: row (i%4) + 4h + 8(i/4), column l%32.
#include "infonce_common.h"

namespace ts {

constexpr int kGenQTile = 128;  // q rows per workgroup (32 per wavefront)
constexpr int kGenKeys = 32;    // keys per LDS tile
constexpr int kGenBlock = 256;
constexpr float kGenFloor = -1.0e30f;  // finite stand-in for "no maximum yet"

struct NceGenLayout {
  int64_t npad;
  int splits, cp;
  size_t head_bytes, off_rq, off_rk, off_stat, off_opart, pair_bytes;
  size_t rowloss_bytes;  // behind the pairs' regions: [pairs][npad] per-row loss terms, summed by the last launch
};

inline int nce_gen_cp(int64_t c) { return c <= 64 ? 64 : (c <= 128 ? 128 : (c <= 256 ? 256 : 512)); }

inline int nce_gen_splits(int64_t npad, int n_pairs, int fgroups, int target) {
  const int64_t wgs = npad / kGenQTile * n_pairs * fgroups;
  const int64_t tiles = npad / kGenKeys;
  int64_t s = (target + wgs - 1) / wgs;
  if (s > 16) s = 16;
  if (s > tiles) s = tiles;
  if (s < 1) s = 1;
  return (int)s;
}

inline int nce_gen_fgroups(int cp) { return cp > 256 ? cp / 128 : 1; }

inline NceGenLayout nce_gen_layout(int64_t n, int64_t c, int n_pairs, int target) {
  NceGenLayout L;
  L.npad = nce_round_up(n > 0 ? n : 1, kGenQTile);
  L.cp = nce_gen_cp(c);
  L.splits = nce_gen_splits(L.npad, n_pairs, nce_gen_fgroups(L.cp), target);
  L.head_bytes = 256;
  size_t o = 0;
  L.off_rq = o;     o += nce_align(L.npad * 4);
  L.off_rk = o;     o += nce_align(L.npad * 4);
  L.off_stat = o;   o += nce_align((size_t)L.splits * L.npad * 16);
  L.off_opart = o;  o += nce_align((size_t)L.splits * L.npad * L.cp * 4);
  L.pair_bytes = o;
  L.rowloss_bytes = nce_align((size_t)n_pairs * L.npad * 4);
  return L;
}

// defined in losses.hip
int launch_sum_scale(const float* v, int64_t n, float scale, float denom, float* out, hipStream_t stream);

// ---------------------------------------------------------------------------
// norm: one wavefront per row
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kGenBlock) void nce_gen_norm_kernel(NceArgs args, int64_t n, int64_t npad, int c) {
  const NcePair& pr = args.p[blockIdx.z];
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  const int64_t row = (int64_t)blockIdx.x * (kGenBlock / kWave) + w;
  if (row >= npad) return;
  float sq = 0.f, sk = 0.f;
  if (row < n) {
    const NceRow rp = nce_row<T>(pr, row, c);
    for (int f = lane; f < c; f += kWave) {
      const float qv = to_f32(((const T*)rp.q)[f]), kv = to_f32(((const T*)rp.k)[f]);
      sq = fmaf(qv, qv, sq);
      sk = fmaf(kv, kv, sk);
    }
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (lane == 0) {
    const bool live = row < n;
    pr.rq[row] = live ? 1.f / fmaxf(sqrtf(sq), kNormEps) : 0.f;
    pr.rk[row] = live ? 1.f / fmaxf(sqrtf(sk), kNormEps) : 0.f;
  }
}

// Four consecutive elements of a row as floats; `vec`: the row is aligned for
// one load of all four (16 bytes of fp32, 8 bytes of a 2-byte type).
template <typename T>
__device__ __forceinline__ void nce_load4(const T* p, int f, int c, bool vec, float (&out)[4]) {
  if (vec && f + 3 < c) {
    T tmp[4];
    __builtin_memcpy(tmp, __builtin_assume_aligned(p + f, 4 * sizeof(T)), sizeof(tmp));
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = to_f32(tmp[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = f + i < c ? to_f32(p[f + i]) : 0.f;
  }
}

// ---------------------------------------------------------------------------
// main
// ---------------------------------------------------------------------------
template <typename T, int CP, int FBW>
__global__ __launch_bounds__(kGenBlock) void nce_gen_main_kernel(NceArgs args, int64_t n, int64_t npad, int c, int splits,
                                                                 float scale2 /* log2(e)/tau */, int vec) {
  constexpr int STRIDE = CP + 1;           // words per key row in LDS
  constexpr int FG = CP / 32 / FBW;        // feature groups (grid z = pair * FG + group)
  constexpr int NU = kGenKeys * CP / 4 / kGenBlock;  // 4-element chunks of a key tile per thread
  static_assert(NU * kGenBlock * 4 == kGenKeys * CP, "tile size");
  __shared__ float kt[2][kGenKeys * STRIDE];
  const NcePair& pr = args.p[blockIdx.z / FG];
  const int fg = blockIdx.z % FG;
  const int tid = threadIdx.x, lane = tid % kWave, w = tid / kWave;
  const int col = lane % 32, h = lane / 32;
  const int64_t qtile = blockIdx.x;
  const int split = blockIdx.y;
  const int64_t qrow = qtile * kGenQTile + w * 32 + col;  // the q row this lane is a column of
  const int tiles = (int)(npad / kGenKeys);
  const int t0 = (int)((int64_t)tiles * split / splits), t1 = (int)((int64_t)tiles * (split + 1) / splits);

  // Q fragments, B operand of S^T: step s = 4j + i contracts feature 8j + 4h + i
  float qf[CP / 2];
  {
    const bool live = qrow < n;
    const T* qp = (const T*)nce_row<T>(pr, live ? qrow : 0, c).q;
#pragma unroll
    for (int j = 0; j < CP / 8; ++j) {
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (live && 8 * j + 4 * h < c) nce_load4<T>(qp, 8 * j + 4 * h, c, vec != 0, v);
#pragma unroll
      for (int i = 0; i < 4; ++i) qf[4 * j + i] = v[i];
    }
  }
  const float rq_i = qrow < n ? pr.rq[qrow] : 0.f;
  const float sc_i = rq_i * scale2;

  // key tile t: global -> registers (normalised on the way), registers -> LDS
  float vst[NU][4];
  auto stage_load = [&](int t) {
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      const int e = (u * kGenBlock + tid) * 4;
      const int key = e / CP, f = e % CP;
      const int64_t row = (int64_t)t * kGenKeys + key;
      vst[u][0] = vst[u][1] = vst[u][2] = vst[u][3] = 0.f;
      if (row < n && f < c) {
        const T* kp = (const T*)nce_row<T>(pr, row, c).k;
        nce_load4<T>(kp, f, c, vec != 0, vst[u]);
        const float rk = pr.rk[row];
#pragma unroll
        for (int i = 0; i < 4; ++i) vst[u][i] *= rk;
      }
    }
  };
  auto stage_store = [&](int buf) {
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      const int e = (u * kGenBlock + tid) * 4;
      const int key = e / CP, f = e % CP;
#pragma unroll
      for (int i = 0; i < 4; ++i) kt[buf][key * STRIDE + f + i] = vst[u][i];
    }
  };

  f32x16 oacc[FBW];
#pragma unroll
  for (int fb = 0; fb < FBW; ++fb)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[fb][i] = 0.f;
  float m_run = kGenFloor;   // running maximum of this q row's logits (log2 domain), shared by the lane pair
  float lneg = 0.f;          // this lane's share of sum_{j != i} 2^(s_ij - m_run)
  float pd = 0.f;            // 2^(s_ii - m_run), on the lane that met the positive key
  float sdiag = -INFINITY;   // s_ii (log2 domain), on the same lane
  // the lane of column col that holds key `col` of a diagonal tile: D register istar, half hstar
  const int hstar = (col >> 2) & 1, istar = (col & 3) + 4 * (col >> 3);
  const int tdiag = (int)(qtile * (kGenQTile / kGenKeys)) + w;  // the tile of this wavefront's own keys

  if (t0 < t1) {
    stage_load(t0);
    stage_store(0);
  }
  __syncthreads();
  for (int t = t0; t < t1; ++t) {
    const int buf = (t - t0) & 1;
    const float* kb = kt[buf];
    if (t + 1 < t1) stage_load(t + 1);

    // S^T[key][q] = sum_f Kh[key][f] Q[q][f].  The A operands of four MFMAs are read from LDS
    // while the four before them run; the order is pinned, because left to itself the compiler
    // issues every read of the tile up front and needs a register for each.
    f32x16 sacc;
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
    const float* ka = kb + col * STRIDE + 4 * h;
    {
      float a_cur[4], a_nxt[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a_cur[i] = ka[i];
#pragma unroll
      for (int j = 0; j < CP / 8; ++j) {
        if (j + 1 < CP / 8) {
#pragma unroll
          for (int i = 0; i < 4; ++i) a_nxt[i] = ka[8 * (j + 1) + i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[i], qf[4 * j + i], sacc, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; ++i) a_cur[i] = a_nxt[i];
      }
    }

    // soft-max against the running maximum; keys beyond the batch get weight zero
    float sv[16];
    const bool ragged = (int64_t)(t + 1) * kGenKeys > n;  // uniform
    float mt = kGenFloor;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      sv[i] = sacc[i] * sc_i;
      if (ragged && (int64_t)t * kGenKeys + (i % 4) + 4 * h + 8 * (i / 4) >= n) sv[i] = -INFINITY;
      mt = fmaxf(mt, sv[i]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 32, kWave));
    const float m_new = fmaxf(m_run, mt);
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    float pv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) pv[i] = fast_exp2(sv[i] - m_new);
    pd *= alpha;
    if (t == tdiag) {  // uniform: the positive key's term leaves the row sum and the second product
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (i == istar && h == hstar) {
          pd = pv[i];
          sdiag = sv[i];
          pv[i] = 0.f;
        }
    }
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) psum += pv[i];
    lneg = fmaf(lneg, alpha, psum);
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
      for (int fb = 0; fb < FBW; ++fb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[fb][i] *= alpha;
    }

    // O^T[f][q] += sum_key Kh[key][f] P[key][q]; step s contracts key (s%4) + 4h + 8(s/4), which is
    // where this lane's pv[s] sits
    const float* kc = kb + 4 * h * STRIDE + 32 * (fg * FBW) + col;
    {
      float a_cur[FBW], a_nxt[FBW];
#pragma unroll
      for (int fb = 0; fb < FBW; ++fb) a_cur[fb] = kc[32 * fb];
#pragma unroll
      for (int s = 0; s < 16; ++s) {
        if (s + 1 < 16) {
#pragma unroll
          for (int fb = 0; fb < FBW; ++fb) a_nxt[fb] = kc[(((s + 1) % 4) + 8 * ((s + 1) / 4)) * STRIDE + 32 * fb];
        }
#pragma unroll
        for (int fb = 0; fb < FBW; ++fb)
          oacc[fb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[fb], pv[s], oacc[fb], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int fb = 0; fb < FBW; ++fb) a_cur[fb] = a_nxt[fb];
      }
    }

    if (t + 1 < t1) stage_store(buf ^ 1);  // last read in iteration t-1, which ended with the barrier below
    __syncthreads();
  }

  // row statistics: the two halves of a lane pair hold different keys of the same q row
  lneg += __shfl_xor(lneg, 32, kWave);
  pd += __shfl_xor(pd, 32, kWave);
  sdiag = fmaxf(sdiag, __shfl_xor(sdiag, 32, kWave));
  if (fg == 0 && h == 0) {
    const f32x4 st = {m_run, lneg, pd, sdiag};
    *reinterpret_cast<f32x4*>(pr.stat + ((int64_t)split * npad + qrow) * 4) = st;
  }
  // partial O as [split][row][CP] fp32: D register group g = i/4 holds features 32 fb + 8 g + 4 h .. +3
  float* op = pr.opart + ((int64_t)split * npad + qrow) * CP + 32 * (fg * FBW) + 4 * h;
#pragma unroll
  for (int fb = 0; fb < FBW; ++fb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 v = {oacc[fb][4 * g], oacc[fb][4 * g + 1], oacc[fb][4 * g + 2], oacc[fb][4 * g + 3]};
      *reinterpret_cast<f32x4*>(op + 32 * fb + 8 * g) = v;
    }
}

// ---------------------------------------------------------------------------
// combine: one wavefront per row.  With w_s = 2^(m_s - M), M = max_s m_s:
//   l_neg = sum_s w_s l_neg,s   p = sum_s w_s p_s   l = l_neg + p
//   O'    = sum_s w_s O'_s
//   dqh   = (2/N) [ O'/l - (l_neg/l) kh_i ]
// Every row also leaves its loss term ln2 (M_i + log2 l_i - s_ii); a last,
// single-workgroup launch adds them up in a fixed order
//   loss = loss_scale / n * sum over pairs and rows.
// ---------------------------------------------------------------------------
struct NceGenRowStat {
  float M, lneg, p, sdiag;
};

constexpr int kGenMaxSplits = 16;  // nce_gen_splits never asks for more

// Every split's record of the row is requested before the first is used.
__device__ __forceinline__ NceGenRowStat nce_gen_merge(const float* stat, int64_t row, int64_t npad, int splits) {
  f32x4 v[kGenMaxSplits];
#pragma unroll
  for (int s = 0; s < kGenMaxSplits; ++s)
    v[s] = s < splits ? *reinterpret_cast<const f32x4*>(stat + ((int64_t)s * npad + row) * 4)
                      : f32x4{kGenFloor, 0.f, 0.f, -INFINITY};
  float M = kGenFloor;
#pragma unroll
  for (int s = 0; s < kGenMaxSplits; ++s) M = fmaxf(M, v[s][0]);
  NceGenRowStat r{M, 0.f, 0.f, -INFINITY};
#pragma unroll
  for (int s = 0; s < kGenMaxSplits; ++s) {
    const float wgt = fast_exp2(v[s][0] - M);
    r.lneg = fmaf(wgt, v[s][1], r.lneg);
    r.p = fmaf(wgt, v[s][2], r.p);
    r.sdiag = fmaxf(r.sdiag, v[s][3]);
  }
  return r;
}

template <typename T>
__global__ __launch_bounds__(kGenBlock) void nce_gen_combine_kernel(NceArgs args, int64_t n, int64_t npad, int c, int cp,
                                                                    int splits, float* __restrict__ rowloss) {
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  const NcePair& pr = args.p[blockIdx.z];
  const int64_t row = (int64_t)blockIdx.x * (kGenBlock / kWave) + w;
  if (row >= npad) return;
  float* const my_loss = rowloss + (int64_t)blockIdx.z * npad + row;
  if (row >= n) {  // padding rows add nothing to the sum
    if (lane == 0) *my_loss = 0.f;
    return;
  }
  const NceRow rp = nce_row<T>(pr, row, c);
  const NceGenRowStat r = nce_gen_merge(pr.stat, row, npad, splits);
  if (lane == 0) *my_loss = kNceLn2 * (r.M + log2f(r.lneg + r.p) - r.sdiag);
  if (!rp.dq) return;
  const float l = r.lneg + r.p;
  const float inv_l = 1.f / l, w_neg = r.lneg * inv_l;
  const float rq_i = pr.rq[row], rk_i = pr.rk[row];
  const float gn = 2.f / (float)n;
  constexpr int MAXF = 512 / kWave;
  constexpr int kMaxSplits = kGenMaxSplits;
  // the splits' weights once, then every partial sum of the row requested before the first is used
  float wgt[kMaxSplits];
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s)
    wgt[s] = s < splits ? fast_exp2(pr.stat[((int64_t)s * npad + row) * 4] - r.M) : 0.f;
  float dqh[MAXF], qh[MAXF];
  float dot = 0.f;
#pragma unroll
  for (int u = 0; u < MAXF; ++u) {
    const int f = u * kWave + lane;
    dqh[u] = qh[u] = 0.f;
    if (u * kWave < c) {  // uniform
      const bool live = f < c;
      float part[kMaxSplits];
#pragma unroll
      for (int s = 0; s < kMaxSplits; ++s)
        part[s] = (live && s < splits) ? pr.opart[((int64_t)s * npad + row) * cp + f] : 0.f;
      const float kv = live ? to_f32(((const T*)rp.k)[f]) : 0.f;
      const float qv = live ? to_f32(((const T*)rp.q)[f]) : 0.f;
      float o = 0.f;
#pragma unroll
      for (int s = 0; s < kMaxSplits; ++s) o = fmaf(wgt[s], part[s], o);
      dqh[u] = gn * (o * inv_l - w_neg * (kv * rk_i));
      qh[u] = qv * rq_i;
      dot = fmaf(qh[u], dqh[u], dot);
    }
  }
  dot = wave_sum(dot);
  // below eps the norm is the constant eps and normalize() is linear: no projection
  if (rq_i >= 1.f / kNormEps) dot = 0.f;
#pragma unroll
  for (int u = 0; u < MAXF; ++u) {
    const int f = u * kWave + lane;
    if (f < c) ((T*)rp.dq)[f] = from_f32<T>((dqh[u] - qh[u] * dot) * rq_i);
  }
}

template <typename T, int CP, int FBW>
int nce_gen_run(const NceArgs& args, int pairs, int64_t n, int c, float tau, const NceGenLayout& L, float* rowloss,
                float* loss_out, bool vec, hipStream_t stream) {
  constexpr int FG = CP / 32 / FBW;
  const unsigned wave_rows = kGenBlock / kWave;
  hipLaunchKernelGGL((nce_gen_norm_kernel<T>), dim3((unsigned)((L.npad + wave_rows - 1) / wave_rows), 1, (unsigned)pairs),
                     dim3(kGenBlock), 0, stream, args, n, L.npad, c);
  int rc = check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL((nce_gen_main_kernel<T, CP, FBW>),
                     dim3((unsigned)(L.npad / kGenQTile), (unsigned)L.splits, (unsigned)(pairs * FG)), dim3(kGenBlock), 0,
                     stream, args, n, L.npad, c, L.splits, kNceLog2e / tau, vec ? 1 : 0);
  rc = check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL((nce_gen_combine_kernel<T>), dim3((unsigned)(L.npad / wave_rows), 1, (unsigned)pairs),
                     dim3(kGenBlock), 0, stream, args, n, L.npad, c, CP, L.splits, rowloss);
  rc = check_launch();
  if (rc) return rc;
  return launch_sum_scale(rowloss, (int64_t)pairs * L.npad, 2.f * tau, (float)n, loss_out, stream);
}

template <typename T>
int nce_gen_dispatch(const NceArgs& args, int pairs, int64_t n, int c, float tau, const NceGenLayout& L, float* rowloss,
                     float* loss_out, bool vec, hipStream_t stream) {
  switch (L.cp) {
    case 64: return nce_gen_run<T, 64, 2>(args, pairs, n, c, tau, L, rowloss, loss_out, vec, stream);
    case 128: return nce_gen_run<T, 128, 4>(args, pairs, n, c, tau, L, rowloss, loss_out, vec, stream);
    case 256: return nce_gen_run<T, 256, 8>(args, pairs, n, c, tau, L, rowloss, loss_out, vec, stream);
    default: return nce_gen_run<T, 512, 4>(args, pairs, n, c, tau, L, rowloss, loss_out, vec, stream);
  }
}

size_t nce_general_workspace_bytes(int64_t n, int64_t c, int n_pairs) {
  const NceGenLayout L = nce_gen_layout(n, c, n_pairs, kNceMaxWorkgroupTarget);
  return L.head_bytes + L.pair_bytes * (size_t)n_pairs + L.rowloss_bytes;
}

int nce_general_launch(NceArgs& args, int pairs, int64_t n, int64_t c, float tau, void* workspace, float* loss_out,
                       int dtype, hipStream_t stream) {
  if (c < 1 || c > 512) return TS_ERR_RANGE;
  const NceGenLayout L = nce_gen_layout(n, c, pairs, nce_workgroup_target());
  char* ws = (char*)workspace;
  const size_t esz = dtype == TS_F32 ? 4 : 2;
  // four elements per load when every row starts on a multiple of that load's size
  bool vec = (c % 4) == 0;
  for (int p = 0; p < 2; ++p) {
    const int src = p < pairs ? p : 0;  // an unused second slot mirrors the first
    if (p >= pairs) args.p[p] = args.p[0];
    char* wsp = ws + L.head_bytes + (size_t)src * L.pair_bytes;
    NcePair& P = args.p[p];
    P.rq = (float*)(wsp + L.off_rq);
    P.rk = (float*)(wsp + L.off_rk);
    P.stat = (float*)(wsp + L.off_stat);
    P.opart = (float*)(wsp + L.off_opart);
    P.pdiag = P.lpart = nullptr;
    P.khat = P.qb = nullptr;
    uintptr_t bits = (uintptr_t)P.q | (uintptr_t)P.k;
    for (int i = 0; i < P.n_pieces; ++i) bits |= (uintptr_t)P.qp[i] | (uintptr_t)P.kp[i];
    if (bits & (4 * esz - 1)) vec = false;
  }
  const int ci = (int)c;
  float* rowloss = (float*)(ws + L.head_bytes + (size_t)pairs * L.pair_bytes);
  if (dtype == TS_F32) return nce_gen_dispatch<float>(args, pairs, n, ci, tau, L, rowloss, loss_out, vec, stream);
  if (dtype == TS_F16) return nce_gen_dispatch<f16_t>(args, pairs, n, ci, tau, L, rowloss, loss_out, vec, stream);
  return nce_gen_dispatch<bf16_t>(args, pairs, n, ci, tau, L, rowloss, loss_out, vec, stream);
}

}  // namespace ts
