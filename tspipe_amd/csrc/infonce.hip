// MoCo-v3 InfoNCE loss, forward and backward fused, on bf16 MFMA.
//
//   qh = q/|q|, kh = k/|k|, logits = qh kh^T / tau,
//   loss = 2 tau * mean_i( lse_i - logits_ii ),
//   dqh_i = (2/N) (sum_j P_ij kh_j - kh_i),  P = softmax(logits) row-wise,
//   dq_i  = (dqh_i - qh_i <qh_i, dqh_i>) / |q_i|.
//
// sum_j P_ij kh_j is an attention product with V = K, so the kernel is a
// flash-attention forward: the N x N logits are never stored.  Two facts make
// it simpler than the general case:
//   * |logit| <= 1/tau because the rows are unit vectors, so the soft-max
//     uses the fixed reference point x_max = log2(e)/tau instead of a running
//     maximum: no rescaling of the accumulators, and partial results of
//     different key ranges just add up;
//   * the normalisation is applied as fp32 factors after the bf16 contraction
//     (logit_ij = <q_i,k_j> * rq_i * rk_j / tau), so the raw bf16 inputs feed
//     the MFMA and no rounded copy of qh / kh is ever made.
//
// Kernels:
//   prep     per row: rq = 1/max(|q|,eps), rk, the diagonal logit, and K^T
//            (bf16, [C][Npad]) so that the second contraction can read keys
//            contiguously; fp32 inputs are also rounded to bf16 copies here.
//   main     grid (q tile of 128 rows, key split, pair); 4 wavefronts, each
//            owning 32 q rows; per 32-key tile: S^T = K Q^T (MFMA 32x32x16),
//            P = 2^(S*scale - x_max), l += P, O^T += K^T (P*rk) (MFMA).
//            Writes per-split partial l and O^T in register-native order.
//   combine  per 32-row q tile: adds the splits, forms loss rows and dq.
//
// MFMA 32x32x16 operand layout used throughout (lane l, half h = l/32):
//   A: row l%32, contraction slots 8h..8h+7;  B: column l%32, same slots;
//   D[i]: row (i%4) + 4h + 8(i/4), column l%32.
#include "common.h"

namespace ts {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr float kNceLog2e = 1.4426950408889634f;
constexpr float kNceLn2 = 0.6931471805599453f;
constexpr float kNormEps = 1e-12f;  // F.normalize's eps
constexpr int kQTile = 128;         // q rows per workgroup (32 per wavefront)
constexpr int kKTile = 32;          // keys per inner iteration
constexpr int kNceBlock = 256;

// defined in losses.hip
int launch_sum_scale(const float* v, int64_t n, float scale, float denom, float* out, hipStream_t stream);

__host__ __device__ inline int64_t nce_round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// Workspace carve-up (all offsets multiples of 256 bytes): a head with the
// loss rows of every pair, [pairs][npad] floats, then one region per pair.
struct NceLayout {
  int64_t npad;
  int splits;
  size_t head_bytes;
  size_t off_rq, off_rk, off_diag, off_lpart, off_apart, off_kt, off_qb, off_kb, off_opart, pair_bytes;
};

inline size_t nce_align(size_t x) { return (x + 255) & ~(size_t)255; }

inline int nce_splits(int64_t npad, int n_pairs) {
  const int64_t qtiles = npad / kQTile * n_pairs;
  const int64_t ktiles = npad / kKTile;
  int64_t s = (256 + qtiles - 1) / qtiles;  // one workgroup per CU: the kernel's registers allow no more
  if (s > 16) s = 16;
  if (s > ktiles) s = ktiles;
  if (s < 1) s = 1;
  return (int)s;
}

inline NceLayout nce_layout(int64_t n, int64_t c, int n_pairs, bool fp32_in) {
  NceLayout L;
  L.npad = nce_round_up(n > 0 ? n : 1, kQTile);
  L.splits = nce_splits(L.npad, n_pairs);
  L.head_bytes = nce_align((size_t)n_pairs * L.npad * 4);
  size_t o = 0;
  L.off_rq = o;       o += nce_align(L.npad * 4);
  L.off_rk = o;       o += nce_align(L.npad * 4);
  L.off_diag = o;     o += nce_align(L.npad * 4);
  L.off_lpart = o;    o += nce_align((size_t)L.splits * L.npad * 4);
  L.off_apart = o;    o += nce_align((size_t)L.splits * L.npad * 4);
  L.off_kt = o;       o += nce_align((size_t)c * L.npad * 2);
  L.off_qb = o;       o += fp32_in ? nce_align((size_t)L.npad * c * 2) : 0;
  L.off_kb = o;       o += fp32_in ? nce_align((size_t)L.npad * c * 2) : 0;
  L.off_opart = o;    o += nce_align((size_t)L.splits * L.npad * c * 4);
  L.pair_bytes = o;
  return L;
}

// ---------------------------------------------------------------------------
// prep: 16-byte row loads, a group of C/VEC lanes per row; the K rows of the
// workgroup pass through LDS to come out transposed
// ---------------------------------------------------------------------------
template <typename T, int C>
struct NcePrep {
  static constexpr int VEC = 16 / sizeof(T);               // elements per 16-byte load
  static constexpr int LPR = C / VEC;                      // lanes per row (8 .. 64)
  static constexpr int RPP = kWave / LPR;                  // rows per wavefront pass
  static constexpr int ROWS = (4 * RPP > 16) ? 4 * RPP : 16;  // rows per workgroup
  static constexpr int LD = C + 8;                         // bf16 per LDS row (16-byte aligned rows)
};

template <typename T, int C>
__global__ __launch_bounds__(kNceBlock) void nce_prep_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                             int64_t n, int64_t npad, float scale2,
                                                             float* __restrict__ rq, float* __restrict__ rk,
                                                             float* __restrict__ diag, uint16_t* __restrict__ kt,
                                                             uint16_t* __restrict__ qb, uint16_t* __restrict__ kb) {
  using P = NcePrep<T, C>;
  __shared__ __attribute__((aligned(16))) uint16_t tile[P::ROWS * P::LD];
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  const int sub = lane / P::LPR, li = lane % P::LPR;  // row within the pass, lane within the row
  const int64_t row0 = (int64_t)blockIdx.x * P::ROWS;

  for (int r = w * P::RPP + sub; r < P::ROWS; r += 4 * P::RPP) {
    const int64_t row = row0 + r;
    const bool live = row < n;
    float qv[P::VEC], kv[P::VEC];
    if (live) {
      u32x4 rawq = *reinterpret_cast<const u32x4*>(q + row * C + li * P::VEC);
      u32x4 rawk = *reinterpret_cast<const u32x4*>(k + row * C + li * P::VEC);
      T tq[P::VEC], tk[P::VEC];
      __builtin_memcpy(tq, &rawq, 16);
      __builtin_memcpy(tk, &rawk, 16);
#pragma unroll
      for (int e = 0; e < P::VEC; ++e) {
        qv[e] = to_f32(tq[e]);
        kv[e] = to_f32(tk[e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < P::VEC; ++e) qv[e] = kv[e] = 0.f;
    }
    float sqq = 0.f, skk = 0.f, sqk = 0.f;
    uint16_t qbits[P::VEC], kbits[P::VEC];
#pragma unroll
    for (int e = 0; e < P::VEC; ++e) {
      qbits[e] = f32_to_bf16_bits(qv[e]);
      kbits[e] = f32_to_bf16_bits(kv[e]);
      sqq += qv[e] * qv[e];
      skk += kv[e] * kv[e];
      // the diagonal logit uses the values the MFMA will see
      sqk += bf16_bits_to_f32(qbits[e]) * bf16_bits_to_f32(kbits[e]);
    }
#pragma unroll
    for (int e = 0; e < P::VEC; ++e) tile[r * P::LD + li * P::VEC + e] = kbits[e];
    if (qb) {
#pragma unroll
      for (int e = 0; e < P::VEC; ++e) {
        qb[row * C + li * P::VEC + e] = qbits[e];
        kb[row * C + li * P::VEC + e] = kbits[e];
      }
    }
#pragma unroll
    for (int off = P::LPR / 2; off > 0; off >>= 1) {
      sqq += __shfl_xor(sqq, off, kWave);
      skk += __shfl_xor(skk, off, kWave);
      sqk += __shfl_xor(sqk, off, kWave);
    }
    if (li == 0) {
      const float a = live ? 1.f / fmaxf(sqrtf(sqq), kNormEps) : 0.f;
      const float b = live ? 1.f / fmaxf(sqrtf(skk), kNormEps) : 0.f;
      rq[row] = a;
      rk[row] = b;
      diag[row] = sqk * a * b * scale2;
    }
  }
  __syncthreads();
  // transposed write: K^T[f][row0 + 8*chunk .. +7], 16 bytes per store
  for (int id = threadIdx.x; id < C * (P::ROWS / 8); id += kNceBlock) {
    const int f = id / (P::ROWS / 8), chunk = id % (P::ROWS / 8);
    u16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = tile[(chunk * 8 + e) * P::LD + f];
    *reinterpret_cast<u16x8*>(kt + (int64_t)f * npad + row0 + chunk * 8) = v;
  }
}

// ---------------------------------------------------------------------------
// main
// ---------------------------------------------------------------------------
template <int C>
struct NceSmem {
  static constexpr int KLD = C + 8;       // bf16 per K-tile row (16-byte pad: rows start on different banks)
  static constexpr int TLD = kKTile + 4;  // bf16 per K^T-tile row: 72 bytes, so 16 consecutive rows start on
                                          // 16 different bank pairs and the 8-byte operand reads do not collide
  uint16_t k[2][kKTile * KLD];
  uint16_t kt[2][C * TLD];
  float rk[2][kKTile];
};

template <int C>
__global__ __launch_bounds__(kNceBlock) void nce_main_kernel(const uint16_t* __restrict__ qg,
                                                             const uint16_t* __restrict__ kg,
                                                             const uint16_t* __restrict__ ktg,
                                                             const float* __restrict__ rq,
                                                             const float* __restrict__ rk, int64_t n, int64_t npad,
                                                             int splits, float scale2 /* log2(e)/tau */,
                                                             float* __restrict__ lpart, float* __restrict__ apart,
                                                             float* __restrict__ opart) {
  using Smem = NceSmem<C>;
  __shared__ __attribute__((aligned(16))) Smem sm;
  constexpr int KK = C / 16;  // contraction steps of S^T
  constexpr int FB = C / 32;  // feature blocks of O^T
  const int tid = threadIdx.x, lane = tid % kWave, w = tid / kWave;
  const int col = lane % 32, h = lane / 32;
  // Workgroup ids are dealt round-robin to the 8 XCDs.  With the key split as
  // the fastest index (and 8 splits), every XCD keeps seeing the same eighth
  // of K and K^T, which then stays in that XCD's own L2.
  const int split = blockIdx.x;
  const int64_t qtile = blockIdx.y;
  const int64_t qrow = qtile * kQTile + w * 32 + col;  // the q row this lane is a column of

  const int64_t ktiles = npad / kKTile;
  const int64_t t0 = ktiles * split / splits, t1 = ktiles * (split + 1) / splits;

  // Q fragments: B operand of S^T, resident for the whole kernel.
  bf16x8 qf[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) {
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (qrow < n) raw = *reinterpret_cast<const u32x4*>(qg + qrow * C + kk * 16 + h * 8);
    __builtin_memcpy(&qf[kk], &raw, 16);
  }
  const float rq_i = (qrow < n) ? rq[qrow] : 0.f;
  const float sc_i = rq_i * scale2;

  f32x16 oacc[FB];
#pragma unroll
  for (int fb = 0; fb < FB; ++fb)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[fb][i] = 0.f;
  float lsum = 0.f;  // sum_j P_ij
  float asum = 0.f;  // sum_j P_ij (x_ij - x_max), x: logit in the log2 domain; x_max * l is added at the end
  // tiles from this one on contain padded keys (never reached when n is a multiple of the tile)
  const int64_t t_pad = n / kKTile;

  // global -> register staging of one key tile (K rows, K^T rows, rk)
  constexpr int KCH = kKTile * C / 8 / kNceBlock;  // 16-byte chunks per thread, K tile
  constexpr int TCH = C * kKTile / 8 / kNceBlock;  // same, K^T tile
  u32x4 stage_k[KCH], stage_t[TCH];
  float stage_rk = 0.f;
  auto load_tile = [&](int64_t t) {
    const int64_t key0 = t * kKTile;
#pragma unroll
    for (int u = 0; u < KCH; ++u) {
      const int id = tid + u * kNceBlock;
      const int r = id / (C / 8), c8 = id % (C / 8);
      u32x4 v = {0u, 0u, 0u, 0u};
      if (key0 + r < n) v = *reinterpret_cast<const u32x4*>(kg + (key0 + r) * C + c8 * 8);
      stage_k[u] = v;
    }
#pragma unroll
    for (int u = 0; u < TCH; ++u) {
      const int id = tid + u * kNceBlock;
      const int f = id / (kKTile / 8), c8 = id % (kKTile / 8);
      stage_t[u] = *reinterpret_cast<const u32x4*>(ktg + (int64_t)f * npad + key0 + c8 * 8);
    }
    if (tid < kKTile) stage_rk = rk[key0 + tid];  // zero for padded keys
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int u = 0; u < KCH; ++u) {
      const int id = tid + u * kNceBlock;
      const int r = id / (C / 8), c8 = id % (C / 8);
      *reinterpret_cast<u32x4*>(&sm.k[buf][r * Smem::KLD + c8 * 8]) = stage_k[u];
    }
#pragma unroll
    for (int u = 0; u < TCH; ++u) {
      const int id = tid + u * kNceBlock;
      const int f = id / (kKTile / 8), c8 = id % (kKTile / 8);
      // rows are only 8-byte aligned: two 8-byte stores
      uint2 lo = {stage_t[u].x, stage_t[u].y}, hi = {stage_t[u].z, stage_t[u].w};
      *reinterpret_cast<uint2*>(&sm.kt[buf][f * Smem::TLD + c8 * 8]) = lo;
      *reinterpret_cast<uint2*>(&sm.kt[buf][f * Smem::TLD + c8 * 8 + 4]) = hi;
    }
    if (tid < kKTile) sm.rk[buf][tid] = stage_rk;
  };

  if (t0 < t1) {
    load_tile(t0);
    store_tile(0);
  }
  __syncthreads();

  for (int64_t t = t0; t < t1; ++t) {
    const int buf = (int)((t - t0) & 1);
    const bool more = t + 1 < t1;
    if (more) load_tile(t + 1);  // in flight while this tile is computed

    // All operand fragments of a phase are read from LDS into their own
    // registers before the phase's MFMAs start: with one wavefront per SIMD
    // nothing else hides the LDS latency, and a read-wait-multiply chain per
    // MFMA would pay it 48 times per tile.
    bf16x8 ka[KK];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(&sm.k[buf][col * Smem::KLD + kk * 16 + h * 8]);
      __builtin_memcpy(&ka[kk], &raw, 16);
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the reads above from being sunk next to their MFMAs
    const f32x4 rk0 = *reinterpret_cast<const f32x4*>(&sm.rk[buf][4 * h]);
    const f32x4 rk1 = *reinterpret_cast<const f32x4*>(&sm.rk[buf][8 + 4 * h]);
    const f32x4 rk2 = *reinterpret_cast<const f32x4*>(&sm.rk[buf][16 + 4 * h]);
    const f32x4 rk3 = *reinterpret_cast<const f32x4*>(&sm.rk[buf][24 + 4 * h]);

    // S^T[key][q] = sum_f K[key][f] Q[q][f]
    f32x16 sacc;
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[kk], qf[kk], sacc, 0, 0, 0);

    // K^T fragments for the second product: issued now, they land while the
    // soft-max arithmetic below runs.  Contraction slot 8h + 4gg + j of step
    // tt is key 16tt + 8gg + 4h + j on both operands.
    bf16x8 ta[FB][2];
#pragma unroll
    for (int fb = 0; fb < FB; ++fb) {
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const uint2* base =
            reinterpret_cast<const uint2*>(&sm.kt[buf][(fb * 32 + col) * Smem::TLD + 16 * tt + 4 * h]);
        const uint2 lo = base[0], hi = base[2];
        const u32x4 raw = {lo.x, lo.y, hi.x, hi.y};
        __builtin_memcpy(&ta[fb][tt], &raw, 16);
      }
    }

    __builtin_amdgcn_sched_barrier(0);

    // P = 2^(S * rq_i * rk_j * log2e/tau - x_max); keys this lane holds:
    // key(i) = (i%4) + 4h + 8(i/4).  With u = x - x_max the kernel sums
    // l = sum P and a' = sum P u; sum P x follows as a' + x_max l at the end.
    float pv[16], uv[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 rk4 = (g == 0) ? rk0 : (g == 1) ? rk1 : (g == 2) ? rk2 : rk3;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = 4 * g + j;
        uv[i] = fmaf(sacc[i], sc_i * rk4[j], -scale2);
        pv[i] = fast_exp2(uv[i]);
      }
    }
    if (t >= t_pad) {
      // padded keys, only at the very end of the key range (their rk is 0,
      // which zeroes the second product, but not the row sums)
      const int keyb = (int)(t * kKTile) + 4 * h;
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (keyb + 8 * (i / 4) + (i % 4) >= (int)n) pv[i] = 0.f;
    }
    bf16x8 pb[2];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 rk4 = (g == 0) ? rk0 : (g == 1) ? rk1 : (g == 2) ? rk2 : rk3;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = 4 * g + j;
        lsum += pv[i];
        asum = fmaf(pv[i], uv[i], asum);
        pb[g / 2][(g % 2) * 4 + j] = (__bf16)(pv[i] * rk4[j]);
      }
    }

    // O^T[f][q] += sum_key K^T[f][key] * (P*rk)[key][q]
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int fb = 0; fb < FB; ++fb)
        oacc[fb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ta[fb][tt], pb[tt], oacc[fb], 0, 0, 0);

    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  // partial results, register-native order: [split][q tile of 32][fb][i][lane]
  const float ltot = lsum + __shfl_xor(lsum, 32, kWave);
  // sum_j P_ij x_ij = <qh_i, sum_j P_ij kh_j> * log2e/tau
  const float atot = asum + __shfl_xor(asum, 32, kWave) + scale2 * ltot;
  if (h == 0) {
    lpart[(int64_t)split * npad + qtile * kQTile + w * 32 + col] = ltot;
    apart[(int64_t)split * npad + qtile * kQTile + w * 32 + col] = atot;
  }
  const int64_t tile32 = qtile * (kQTile / 32) + w;
  float* op = opart + (((int64_t)split * (npad / 32) + tile32) * FB) * 16 * kWave;
#pragma unroll
  for (int fb = 0; fb < FB; ++fb)
#pragma unroll
    for (int i = 0; i < 16; ++i) op[(fb * 16 + i) * kWave + lane] = oacc[fb][i];
}

// ---------------------------------------------------------------------------
// combine: one wavefront per (32 q rows, 32-feature block); purely
// element-wise, because <qh_i, dqh_i> follows from the row sums:
//   <qh_i, sum_j P_ij kh_j> = (tau/log2e) A_i / l_i,  <qh_i, kh_i> = (tau/log2e) diag_i
// ---------------------------------------------------------------------------
template <typename T, int C>
__global__ __launch_bounds__(kNceBlock) void nce_combine_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                                const float* __restrict__ rq,
                                                                const float* __restrict__ rk,
                                                                const float* __restrict__ diag,
                                                                const float* __restrict__ lpart,
                                                                const float* __restrict__ apart,
                                                                const float* __restrict__ opart, int64_t n,
                                                                int64_t npad, int splits, float scale2,
                                                                float* __restrict__ row_loss, T* __restrict__ dq) {
  constexpr int FB = C / 32;
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  const int col = lane % 32, h = lane / 32;
  const int64_t item = (int64_t)blockIdx.x * (kNceBlock / kWave) + w;
  const int64_t tile32 = item / FB;
  const int fb = (int)(item % FB);
  if (tile32 >= npad / 32) return;
  const int64_t row = tile32 * 32 + col;
  const bool live = row < n;

  float l = 0.f, A = 0.f;
  for (int s = 0; s < splits; ++s) {
    l += lpart[(int64_t)s * npad + row];
    A += apart[(int64_t)s * npad + row];
  }
  const float d = diag[row];
  if (fb == 0 && h == 0) row_loss[row] = live ? kNceLn2 * (scale2 + log2f(l) - d) : 0.f;
  if (!dq) return;

  float o[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) o[i] = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float* op = opart + (((int64_t)s * (npad / 32) + tile32) * FB + fb) * 16 * kWave;
#pragma unroll
    for (int i = 0; i < 16; ++i) o[i] += op[i * kWave + lane];
  }
  if (!live) return;
  const float inv_l = 1.f / l;
  const float rq_i = rq[row], rk_i = rk[row];
  const float gn = 2.f / (float)n;
  // below eps the norm is the constant eps and normalize() is linear: no projection
  const bool clamped = rq_i >= 1.f / kNormEps;
  const float dot = clamped ? 0.f : gn * (A * inv_l - d) / scale2;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int f0 = 32 * fb + 8 * g + 4 * h;  // this lane holds features f0 .. f0+3 of its row
    T kv[4], qv[4], out[4];
    __builtin_memcpy(kv, k + row * C + f0, sizeof(kv));
    __builtin_memcpy(qv, q + row * C + f0, sizeof(qv));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float dqh = gn * (o[4 * g + j] * inv_l - to_f32(kv[j]) * rk_i);
      out[j] = from_f32<T>((dqh - to_f32(qv[j]) * rq_i * dot) * rq_i);
    }
    __builtin_memcpy(dq + row * C + f0, out, sizeof(out));
  }
}

template <typename T, int C>
int nce_run_pair(const void* q, const void* k, void* dq, int64_t n, float tau, char* ws, float* row_loss,
                 const NceLayout& L, hipStream_t stream) {
  constexpr bool kF32 = sizeof(T) == 4;
  float* rq = (float*)(ws + L.off_rq);
  float* rk = (float*)(ws + L.off_rk);
  float* diag = (float*)(ws + L.off_diag);
  float* lpart = (float*)(ws + L.off_lpart);
  float* apart = (float*)(ws + L.off_apart);
  uint16_t* kt = (uint16_t*)(ws + L.off_kt);
  uint16_t* qb = kF32 ? (uint16_t*)(ws + L.off_qb) : nullptr;
  uint16_t* kb = kF32 ? (uint16_t*)(ws + L.off_kb) : nullptr;
  float* opart = (float*)(ws + L.off_opart);
  const float scale2 = kNceLog2e / tau;

  hipLaunchKernelGGL((nce_prep_kernel<T, C>), dim3((unsigned)(L.npad / NcePrep<T, C>::ROWS)), dim3(kNceBlock), 0,
                     stream, (const T*)q, (const T*)k, n, L.npad, scale2, rq, rk, diag, kt, qb, kb);
  int rc = check_launch();
  if (rc) return rc;
  const uint16_t* qsrc = kF32 ? qb : (const uint16_t*)q;
  const uint16_t* ksrc = kF32 ? kb : (const uint16_t*)k;
  // with bf16 copies the rows beyond n exist (zero); the kernel guards by n either way
  hipLaunchKernelGGL((nce_main_kernel<C>), dim3((unsigned)L.splits, (unsigned)(L.npad / kQTile)),
                     dim3(kNceBlock), 0, stream, qsrc, ksrc, kt, rq, rk, n, L.npad, L.splits, scale2, lpart,
                     apart, opart);
  rc = check_launch();
  if (rc) return rc;
  const int64_t items = L.npad / 32 * (C / 32);  // a multiple of 4: npad is a multiple of 128
  hipLaunchKernelGGL((nce_combine_kernel<T, C>), dim3((unsigned)(items / 4)), dim3(kNceBlock), 0, stream,
                     (const T*)q, (const T*)k, rq, rk, diag, lpart, apart, opart, n, L.npad, L.splits, scale2,
                     row_loss, (T*)dq);
  return check_launch();
}

template <typename T>
int nce_dispatch_c(const void* q, const void* k, void* dq, int64_t n, int64_t c, float tau, char* ws,
                   float* row_loss, const NceLayout& L, hipStream_t stream) {
  switch (c) {
    case 64: return nce_run_pair<T, 64>(q, k, dq, n, tau, ws, row_loss, L, stream);
    case 128: return nce_run_pair<T, 128>(q, k, dq, n, tau, ws, row_loss, L, stream);
    case 256: return nce_run_pair<T, 256>(q, k, dq, n, tau, ws, row_loss, L, stream);
    default: return TS_ERR_ARG;
  }
}

}  // namespace ts

extern "C" {

size_t ts_infonce_workspace_bytes(int64_t n, int64_t c, int n_pairs) {
  if (n < 0 || c <= 0 || n_pairs < 1 || n_pairs > 2) return 0;
  // sized for fp32 inputs (the larger layout) so one query serves both dtypes
  const ts::NceLayout L = ts::nce_layout(n, c, n_pairs, true);
  return L.head_bytes + L.pair_bytes * (size_t)n_pairs;
}

int ts_infonce_fwd_bwd(const void* q1, const void* k1, const void* q2, const void* k2, int64_t n, int64_t c,
                       float tau, void* workspace, float* loss_out, void* dq1, void* dq2, int dtype,
                       ts_stream_t stream) {
  if (!q1 || !k1 || !workspace || !loss_out) return TS_ERR_ARG;
  if ((q2 == nullptr) != (k2 == nullptr)) return TS_ERR_ARG;
  if (n < 0 || !(tau > 0.f)) return TS_ERR_ARG;
  if (c != 64 && c != 128 && c != 256) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16) return TS_ERR_ARG;
  // fixed soft-max reference point: 2^(-2 log2(e)/tau) must stay a normal fp32
  if (tau < 0.03f) return TS_ERR_RANGE;
  if (n > (1 << 24)) return TS_ERR_RANGE;
  if ((uintptr_t)workspace & 255u) return TS_ERR_ALIGN;
  // rows are read as 16-byte vectors
  if (((uintptr_t)q1 | (uintptr_t)k1 | (uintptr_t)q2 | (uintptr_t)k2) & 15u) return TS_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const int pairs = q2 ? 2 : 1;
  if (n == 0) {
    // cross entropy over zero rows: mean of nothing = NaN, as torch gives
    return ts::launch_sum_scale((const float*)workspace, 0, 1.f, 0.f, loss_out, st);
  }
  const ts::NceLayout L = ts::nce_layout(n, c, pairs, true);
  char* ws = (char*)workspace;
  float* row_loss = (float*)ws;
  for (int p = 0; p < pairs; ++p) {
    const void* q = p ? q2 : q1;
    const void* k = p ? k2 : k1;
    void* dq = p ? dq2 : dq1;
    char* wsp = ws + L.head_bytes + (size_t)p * L.pair_bytes;
    float* rl = row_loss + (size_t)p * L.npad;
    int rc = (dtype == TS_F32) ? ts::nce_dispatch_c<float>(q, k, dq, n, c, tau, wsp, rl, L, st)
                               : ts::nce_dispatch_c<ts::bf16_t>(q, k, dq, n, c, tau, wsp, rl, L, st);
    if (rc) return rc;
  }
  // loss = 2 tau / n * sum over all pairs' rows (padding rows hold zero)
  return ts::launch_sum_scale(row_loss, (int64_t)pairs * L.npad, 2.f * tau, (float)n, loss_out, st);
}

}  // extern "C"
