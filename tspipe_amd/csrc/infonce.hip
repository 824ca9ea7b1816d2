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
//   * the keys are normalised in fp32 and rounded to bf16 once, by the prep
//     kernel (the tile images below hold kh); the queries feed the MFMA as
//     they are (bf16 inputs in place, fp32 / fp16 inputs through a bf16 copy)
//     and their 1/|q| is applied as an fp32 factor after the contraction
//     (logit_ij = <q_i, kh_j> * rq_i / tau).
//
// Kernels:
//   prep     per row: rq = 1/max(|q|,eps), rk, the diagonal logit; the keys,
//            normalised and rounded to bf16, are written as "tile images":
//            for every 32 keys the exact bytes, in the exact order, that the
//            main kernel's MFMA operand reads want to find in LDS (below).
//            fp32 and fp16 queries are also rounded to a bf16 copy here.
//   main     grid (q tile of 128 rows, key split); 4 wavefronts, each owning
//            32 q rows; per 32-key tile: S^T = Kh Q^T (MFMA 32x32x16),
//            P = 2^(S*scale - x_max), l += P, O^T += Kh^T P (MFMA).  Tile
//            images go from global memory straight into LDS (no registers),
//            three tiles ahead.  Writes per-split partial l and O^T in
//            register-native order.
//   combine  per 32-row q tile: adds the splits and forms dq; its first
//            workgroup adds up the loss from the split row sums.
//
// Tile image (C features, KK = C/16, FB = C/32; 1 KB fragments, lane L =
// 32h + col reads bytes 16L..16L+15 of a fragment as one MFMA A operand):
//   fragment kk < KK        : Kh[key = col][16kk + 8h .. +7]       (first product)
//   fragment KK + tt*FB + fb: Kh[16tt + 8gg + 4h + j][32fb + col],  (second product)
//                             gg = 0,1, j = 0..3 -> element 4gg + j
// so every operand read is a linear, conflict-free 1 KB of LDS.
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

// Workspace carve-up (all offsets multiples of 256 bytes): a small head, then
// one region per pair.
struct NceLayout {
  int64_t npad;
  int splits;
  size_t head_bytes;
  size_t off_rq, off_rk, off_diag, off_lpart, off_apart, off_kimg, off_qb, off_opart, pair_bytes;
};

// One (q, k) pair's pointers; the kernels pick theirs by blockIdx.z, so the two
// pairs of the symmetric loss share every launch.
struct NcePair {
  const void* q;
  const void* k;
  void* dq;
  const uint16_t* qsrc;  // bf16 queries the MFMA reads: q itself or the rounded copy
  float *rq, *rk, *diag, *lpart, *apart, *opart;
  uint8_t* kimg;
  uint16_t* qb;
};
struct NceArgs {
  NcePair p[2];
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
  L.head_bytes = 256;  // scratch for the empty-batch case
  size_t o = 0;
  L.off_rq = o;       o += nce_align(L.npad * 4);
  L.off_rk = o;       o += nce_align(L.npad * 4);
  L.off_diag = o;     o += nce_align(L.npad * 4);
  L.off_lpart = o;    o += nce_align((size_t)L.splits * L.npad * 4);
  L.off_apart = o;    o += nce_align((size_t)L.splits * L.npad * 4);
  L.off_kimg = o;     o += nce_align((size_t)L.npad * c * 4);  // npad/32 tile images of 128 c bytes
  L.off_qb = o;       o += fp32_in ? nce_align((size_t)L.npad * c * 2) : 0;
  L.off_opart = o;    o += nce_align((size_t)L.splits * L.npad * c * 4);
  L.pair_bytes = o;
  return L;
}

// ---------------------------------------------------------------------------
// prep: 16-byte row loads, a group of C/VEC lanes per row; one workgroup per
// 32 rows, whose normalised keys pass through LDS to come out as a tile image
// ---------------------------------------------------------------------------
template <int C>
struct NceTile {
  static constexpr int KK = C / 16;             // contraction steps of S^T = fragments of the first product
  static constexpr int FB = C / 32;             // feature blocks of O^T
  static constexpr int FRAGS = KK + 2 * FB;     // 1 KB fragments per image
  static constexpr int BYTES = FRAGS * 1024;    // 32 KB at C = 256
};

template <typename T, int C>
struct NcePrep {
  static constexpr int VEC = 16 / sizeof(T);  // elements per 16-byte load
  static constexpr int LPR = C / VEC;         // lanes per row (8 .. 64)
  static constexpr int RPP = kWave / LPR;     // rows per wavefront pass
  static constexpr int ROWS = kKTile;         // rows per workgroup: one key tile
  static constexpr int LD = C + 8;            // bf16 per LDS row (16-byte aligned rows)
};

template <typename T, int C>
__global__ __launch_bounds__(kNceBlock) void nce_prep_kernel(NceArgs args, int64_t n, int64_t npad, float scale2) {
  const NcePair& pr = args.p[blockIdx.z];
  const T* __restrict__ q = (const T*)pr.q;
  const T* __restrict__ k = (const T*)pr.k;
  float* __restrict__ rq = pr.rq;
  float* __restrict__ rk = pr.rk;
  float* __restrict__ diag = pr.diag;
  uint8_t* __restrict__ kimg = pr.kimg;
  uint16_t* __restrict__ qb = pr.qb;
  using P = NcePrep<T, C>;
  using TI = NceTile<C>;
  __shared__ __attribute__((aligned(16))) uint16_t tile[P::ROWS * P::LD];
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  const int sub = lane / P::LPR, li = lane % P::LPR;  // row within the pass, lane within the row
  const int64_t row0 = (int64_t)blockIdx.x * P::ROWS;

  // the loads of all of this wavefront's rows go out before any is used
  constexpr int NP = P::ROWS / (4 * P::RPP);  // passes (rows per lane group)
  static_assert(NP >= 1 && NP * 4 * P::RPP == P::ROWS, "rows divide evenly among the wavefronts");
  u32x4 rawq[NP], rawk[NP];
#pragma unroll
  for (int pass = 0; pass < NP; ++pass) {
    const int64_t row = row0 + w * P::RPP + sub + pass * 4 * P::RPP;
    rawq[pass] = rawk[pass] = u32x4{0u, 0u, 0u, 0u};  // zero rows beyond n (0.0 in every dtype)
    if (row < n) {
      rawq[pass] = *reinterpret_cast<const u32x4*>(q + row * C + li * P::VEC);
      rawk[pass] = *reinterpret_cast<const u32x4*>(k + row * C + li * P::VEC);
    }
  }
#pragma unroll
  for (int pass = 0; pass < NP; ++pass) {
    const int r = w * P::RPP + sub + pass * 4 * P::RPP;
    const int64_t row = row0 + r;
    const bool live = row < n;
    float qv[P::VEC], kv[P::VEC];
    {
      T tq[P::VEC], tk[P::VEC];
      __builtin_memcpy(tq, &rawq[pass], 16);
      __builtin_memcpy(tk, &rawk[pass], 16);
#pragma unroll
      for (int e = 0; e < P::VEC; ++e) {
        qv[e] = to_f32(tq[e]);
        kv[e] = to_f32(tk[e]);
      }
    }
    float sqq = 0.f, skk = 0.f;
#pragma unroll
    for (int e = 0; e < P::VEC; ++e) {
      sqq += qv[e] * qv[e];
      skk += kv[e] * kv[e];
    }
#pragma unroll
    for (int off = P::LPR / 2; off > 0; off >>= 1) {
      sqq += __shfl_xor(sqq, off, kWave);
      skk += __shfl_xor(skk, off, kWave);
    }
    const float a = live ? 1.f / fmaxf(sqrtf(sqq), kNormEps) : 0.f;
    const float b = live ? 1.f / fmaxf(sqrtf(skk), kNormEps) : 0.f;
    // the diagonal logit uses the values the MFMA will see: q rounded to
    // bf16, k normalised and then rounded
    float sqk = 0.f;
    uint16_t qbits[P::VEC];
#pragma unroll
    for (int e = 0; e < P::VEC; ++e) {
      qbits[e] = f32_to_bf16_bits(qv[e]);
      const uint16_t kbits = f32_to_bf16_bits(kv[e] * b);
      tile[r * P::LD + li * P::VEC + e] = kbits;
      sqk += bf16_bits_to_f32(qbits[e]) * bf16_bits_to_f32(kbits);
    }
    if (qb) {
#pragma unroll
      for (int e = 0; e < P::VEC; ++e) qb[row * C + li * P::VEC + e] = qbits[e];
    }
#pragma unroll
    for (int off = P::LPR / 2; off > 0; off >>= 1) sqk += __shfl_xor(sqk, off, kWave);
    if (li == 0) {
      rq[row] = a;
      rk[row] = b;
      diag[row] = sqk * a * scale2;
    }
  }
  __syncthreads();
  // the tile image, 16 bytes per store, consecutive threads -> consecutive chunks
  uint8_t* img = kimg + (int64_t)blockIdx.x * TI::BYTES;
  for (int id = threadIdx.x; id < TI::FRAGS * kWave; id += kNceBlock) {
    const int fr = id / kWave, L = id % kWave;
    const int col = L % 32, h = L / 32;
    u16x8 v;
    if (fr < TI::KK) {
      v = *reinterpret_cast<const u16x8*>(&tile[col * P::LD + fr * 16 + h * 8]);
    } else {
      const int tt = (fr - TI::KK) / TI::FB, fb = (fr - TI::KK) % TI::FB;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = tile[(16 * tt + 8 * (e / 4) + 4 * h + (e % 4)) * P::LD + fb * 32 + col];
    }
    *reinterpret_cast<u16x8*>(img + (int64_t)id * 16) = v;
  }
}

// ---------------------------------------------------------------------------
// main
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void nce_lds_void;
typedef __attribute__((address_space(1))) const void nce_glb_void;
constexpr int kNceBufs = 4;  // tile images in LDS: two in use (tiles t, t+1), two on their way

template <int C>
__global__ __launch_bounds__(kNceBlock) void nce_main_kernel(NceArgs args, int64_t n, int64_t npad, int splits,
                                                             float scale2 /* log2(e)/tau */, int qtile_major) {
  const NcePair& pr = args.p[blockIdx.z];
  const uint16_t* __restrict__ qg = pr.qsrc;
  const uint8_t* __restrict__ kimg = pr.kimg;
  const float* __restrict__ rq = pr.rq;
  float* __restrict__ lpart = pr.lpart;
  float* __restrict__ apart = pr.apart;
  float* __restrict__ opart = pr.opart;
  using TI = NceTile<C>;
  constexpr int KK = TI::KK, FB = TI::FB;
  __shared__ __attribute__((aligned(16))) uint8_t sm[kNceBufs][TI::BYTES];
  const int tid = threadIdx.x, lane = tid % kWave, w = tid / kWave;
  const int col = lane % 32, h = lane / 32;
  // Workgroup ids are dealt round-robin to the 8 XCDs.  While all key images
  // fit an XCD's L2 (4 MB at N = 4096), the q tile is the fastest index: the
  // key splits of a q tile run on one XCD, which streams every image through
  // its L2 (measured 5 % faster there).  For more keys the split is the
  // fastest index, so that an XCD keeps seeing the same share of the images.
  const int split = qtile_major ? blockIdx.y : blockIdx.x;
  const int64_t qtile = qtile_major ? blockIdx.x : blockIdx.y;
  const int64_t qrow = qtile * kQTile + w * 32 + col;  // the q row this lane is a column of

  const int64_t ktiles = npad / kKTile;
  const int64_t t0 = ktiles * split / splits, t1 = ktiles * (split + 1) / splits;

  // Global -> LDS without passing through registers: every wavefront moves a
  // quarter of the image, 1 KB (16 bytes per lane) per instruction, and the
  // hardware writes lane L's bytes at (LDS base) + 16 L, which is exactly
  // the image's own order.  Completion is the issuing wavefront's vector
  // memory counter; the barrier after it makes all four quarters visible.
  constexpr int FPW = TI::FRAGS / 4;  // fragments per wavefront
  auto fetch_tile = [&](int64_t t, int buf) {
    const uint8_t* src = kimg + t * TI::BYTES + (w * FPW) * 1024 + lane * 16;
#pragma unroll
    for (int u = 0; u < FPW; ++u)
      __builtin_amdgcn_global_load_lds((nce_glb_void*)(src + u * 1024),
                                       (nce_lds_void*)(&sm[buf][(w * FPW + u) * 1024]), 16, 0, 0);
  };
  auto wait_fetches_and_sync = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's fetches have landed
    __syncthreads();
  };

  if (t0 < t1) fetch_tile(t0, 0);
  if (t0 + 1 < t1) fetch_tile(t0 + 1, 1);
  if (t0 + 2 < t1) fetch_tile(t0 + 2, 2);

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

  // The loop is software-pipelined so that the matrix pipe and the vector
  // ALU work at the same time: tile t+1's first product is issued before
  // tile t's soft-max, whose exponentials then run while those MFMAs execute.
  // Operand fragments are read from LDS a phase ahead of their MFMAs for the
  // same reason: tile t's K^T fragments while tile t+1's first product runs,
  // tile t+2's K fragments while tile t's second product runs.
  bf16x8 ka[KK];
  auto read_ka = [&](int buf) {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(&sm[buf][kk * 1024 + lane * 16]);
      __builtin_memcpy(&ka[kk], &raw, 16);
    }
  };
  // S^T[key][q] = sum_f Kh[key][f] Q[q][f], as two independent accumulation
  // chains: a dependent MFMA waits for its predecessor's result.
  struct SAcc {
    f32x16 a, b;
  };
  auto first_product = [&](SAcc& s) {
#pragma unroll
    for (int i = 0; i < 16; ++i) s.a[i] = s.b[i] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KK; kk += 2) {
      s.a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[kk], qf[kk], s.a, 0, 0, 0);
      s.b = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[kk + 1], qf[kk + 1], s.b, 0, 0, 0);
    }
  };

  int cur = 0;  // buffer of tile t
  auto next_buf = [](int b) { return b == kNceBufs - 1 ? 0 : b + 1; };

  // One tile; sa holds S^T of tile t on entry, sb receives tile t+1's.
  auto step = [&](int64_t t, const SAcc& sa, SAcc& sb) {
    const int b1 = next_buf(cur), b2 = next_buf(b1), b3 = next_buf(b2);
    // After this barrier tile t+2 is complete in LDS (its fetches were issued
    // a whole tile ago) and every wavefront has finished reading tile t-1,
    // whose buffer the fetch below overwrites.
    wait_fetches_and_sync();

    // no branch (one would split the scheduling regions below): near the end
    // the fetch repeats the last tile into a buffer nobody reads any more
    fetch_tile(t + 3 < ktiles ? t + 3 : ktiles - 1, b3);
    __builtin_amdgcn_sched_barrier(0);

    // Phase 1: tile t+1's first product; in its shadow tile t's soft-max and
    // the reads of tile t's K^T fragments, which take over the registers of
    // the K fragments as the MFMAs release them.
    first_product(sb);  // stale operands after the last tile: result unused
    bf16x8 ta[2 * FB];
#pragma unroll
    for (int x = 0; x < 2 * FB; ++x) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(&sm[cur][(KK + x) * 1024 + lane * 16]);
      __builtin_memcpy(&ta[x], &raw, 16);
    }
    // P = 2^(S * rq_i * log2e/tau - x_max); keys this lane holds:
    // key(i) = (i%4) + 4h + 8(i/4).  With u = x - x_max the kernel sums
    // l = sum P and a' = sum P u; sum P x follows as a' + x_max l at the end.
    float pv[16], uv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      uv[i] = fmaf(sa.a[i] + sa.b[i], sc_i, -scale2);
      pv[i] = fast_exp2(uv[i]);
    }
    bf16x8 pb[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      lsum += pv[i];
      asum = fmaf(pv[i], uv[i], asum);
      pb[i / 8][i % 8] = (__bf16)pv[i];
    }
    // An MFMA occupies the matrix pipe for tens of cycles, but the wavefront
    // issues in order: only instructions placed between two MFMAs run in
    // their shadow.  Ask the scheduler for that interleaving.
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                    // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, (2 * FB + KK - 1) / KK, 0);  // LDS reads
      __builtin_amdgcn_sched_group_barrier(0x002, (112 + KK - 1) / KK, 0);  // its share of the soft-max
    }
    __builtin_amdgcn_sched_barrier(0);

    // Phase 2: O^T[f][q] += sum_key Kh^T[f][key] * P[key][q]; contraction slot
    // 8h + 4gg + j of step tt is key 16tt + 8gg + 4h + j on both operands.
    // In its shadow the reads of tile t+2's K fragments (stale bytes near the
    // end, never used), into the registers the K^T fragments release.
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int fb = 0; fb < FB; ++fb)
        oacc[fb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ta[tt * FB + fb], pb[tt], oacc[fb], 0, 0, 0);
    read_ka(b2);
#pragma unroll
    for (int x = 0; x < 2 * FB; ++x) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, (KK + 2 * FB - 1) / (2 * FB), 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    cur = b1;
  };

  // prologue: S^T of the first tile, K fragments of the second
  SAcc sx, sy;
  wait_fetches_and_sync();
  read_ka(0);
  first_product(sx);
  __builtin_amdgcn_sched_barrier(0);
  read_ka(1);
  __builtin_amdgcn_sched_barrier(0);

  // two tiles per trip, so that the S^T registers alternate without copies
  for (int64_t t = t0; t < t1; t += 2) {
    step(t, sx, sy);
    if (t + 1 < t1) step(t + 1, sy, sx);
  }

  // The last trips fetched tiles nobody reads; they must have landed before
  // this workgroup's LDS can be handed to another one.
  __builtin_amdgcn_s_waitcnt(0x0f70);

  // Padded keys (image rows of zeros) took part in the row sums with the same
  // term for every row, 2^(0 - x_max); take this lane's share of them out.
  {
    int cnt = 0;
    for (int64_t t = (t0 > t_pad ? t0 : t_pad); t < t1; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) cnt += (t * kKTile + 4 * h + 8 * (i / 4) + (i % 4) >= n) ? 1 : 0;
    const float u0 = fmaf(0.f, sc_i, -scale2);
    const float c0 = (float)cnt * fast_exp2(u0);
    lsum -= c0;
    asum = fmaf(-c0, u0, asum);
  }

  // partial results in register-native order
  const float ltot = lsum + __shfl_xor(lsum, 32, kWave);
  // sum_j P_ij x_ij = <qh_i, sum_j P_ij kh_j> * log2e/tau
  const float atot = asum + __shfl_xor(asum, 32, kWave) + scale2 * ltot;
  if (h == 0) {
    lpart[(int64_t)split * npad + qtile * kQTile + w * 32 + col] = ltot;
    apart[(int64_t)split * npad + qtile * kQTile + w * 32 + col] = atot;
  }
  const int64_t tile32 = qtile * (kQTile / 32) + w;
  // [split][q tile of 32][fb][i/4][lane][i%4]: 16 bytes per lane and store
  f32x4* op = reinterpret_cast<f32x4*>(opart + (((int64_t)split * (npad / 32) + tile32) * FB) * 16 * kWave);
#pragma unroll
  for (int fb = 0; fb < FB; ++fb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 v = {oacc[fb][4 * g], oacc[fb][4 * g + 1], oacc[fb][4 * g + 2], oacc[fb][4 * g + 3]};
      op[(fb * 4 + g) * kWave + lane] = v;
    }
}

// ---------------------------------------------------------------------------
// combine: one wavefront per (32 q rows, 32-feature block); purely
// element-wise, because <qh_i, dqh_i> follows from the row sums:
//   <qh_i, sum_j P_ij kh_j> = (tau/log2e) A_i / l_i,  <qh_i, kh_i> = (tau/log2e) diag_i
// ---------------------------------------------------------------------------
// The scalar loss, by one workgroup straight from the split row sums:
//   loss = loss_scale / n * sum over pairs and rows of ln2 (x_max + log2 l_i - diag_i).
// Re-deriving l_i here instead of reading the other workgroups' results keeps
// the reduction inside this launch; the order of every addition is fixed.
__device__ __forceinline__ void nce_loss_block(const NceArgs& args, int pairs, int64_t n, int64_t npad, int splits,
                                               float scale2, float loss_scale, float* __restrict__ loss_out) {
  __shared__ float red[kNceBlock / kWave];
  const int tid = threadIdx.x;
  constexpr int U = 4;   // row quads per thread and trip
  constexpr int SC = 4;  // splits per batch of loads
  const int64_t quads = npad / 4;
  float acc = 0.f;
  for (int p = 0; p < pairs; ++p) {
    const float* __restrict__ lpart = args.p[p].lpart;
    const float* __restrict__ diag = args.p[p].diag;
    for (int64_t q0 = tid; q0 < quads; q0 += (int64_t)U * kNceBlock) {
      // Loads of a batch are all issued before the first is used; a quad or a
      // split beyond the end re-reads a valid address and is added as zero, so
      // no branch separates the loads.
      int64_t quad[U];
      float keep_q[U];
      f32x4 l[U], d[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t want = q0 + (int64_t)u * kNceBlock;
        keep_q[u] = want < quads ? 1.f : 0.f;
        quad[u] = want < quads ? want : q0;
        l[u] = f32x4{0.f, 0.f, 0.f, 0.f};
        d[u] = *reinterpret_cast<const f32x4*>(diag + 4 * quad[u]);
      }
      for (int s0 = 0; s0 < splits; s0 += SC) {
        f32x4 v[SC][U];
        float keep_s[SC];
#pragma unroll
        for (int c = 0; c < SC; ++c) {
          keep_s[c] = s0 + c < splits ? 1.f : 0.f;
          const int sp = s0 + c < splits ? s0 + c : s0;
#pragma unroll
          for (int u = 0; u < U; ++u) v[c][u] = *reinterpret_cast<const f32x4*>(lpart + (int64_t)sp * npad + 4 * quad[u]);
        }
#pragma unroll
        for (int c = 0; c < SC; ++c)
#pragma unroll
          for (int u = 0; u < U; ++u) l[u] += v[c][u] * keep_s[c];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bool live = keep_q[u] != 0.f && 4 * quad[u] + j < n;
          const float term = kNceLn2 * (scale2 + log2f(l[u][j]) - d[u][j]);
          acc += live ? term : 0.f;
        }
      }
    }
  }
  acc = wave_sum(acc);
  if (tid % kWave == 0) red[tid / kWave] = acc;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < kNceBlock / kWave; ++w) total += red[w];
    *loss_out = total * loss_scale / (float)n;
  }
}

template <typename T, int C>
__global__ __launch_bounds__(kNceBlock) void nce_combine_kernel(NceArgs args, int64_t n, int64_t npad, int splits,
                                                                float scale2, float loss_scale,
                                                                float* __restrict__ loss_out) {
  // workgroup 0 of the first pair computes the loss; the (q tile, feature block) items start at workgroup 1
  if (blockIdx.x == 0) {
    if (blockIdx.z == 0) nce_loss_block(args, (int)gridDim.z, n, npad, splits, scale2, loss_scale, loss_out);
    return;
  }
  const NcePair& pr = args.p[blockIdx.z];
  const T* __restrict__ q = (const T*)pr.q;
  const T* __restrict__ k = (const T*)pr.k;
  const float* __restrict__ rq = pr.rq;
  const float* __restrict__ rk = pr.rk;
  const float* __restrict__ diag = pr.diag;
  const float* __restrict__ lpart = pr.lpart;
  const float* __restrict__ apart = pr.apart;
  const float* __restrict__ opart = pr.opart;
  T* __restrict__ dq = (T*)pr.dq;
  constexpr int FB = C / 32;
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  const int col = lane % 32, h = lane / 32;
  const int64_t item = (int64_t)(blockIdx.x - 1) * (kNceBlock / kWave) + w;
  const int64_t tile32 = item / FB;
  const int fb = (int)(item % FB);
  if (tile32 >= npad / 32) return;
  const int64_t row = tile32 * 32 + col;
  const bool live = row < n;

  // The kernel is bound by memory latency, not by arithmetic: every load whose
  // address is known up front is issued before the first use of any of them
  // (the row sums, the k and q values of this lane, the first four splits of
  // the partial O^T).
  const int64_t qk_row = live ? row : 0;  // padded rows read row 0 and discard it
  T kv[4][4], qv[4][4];
  if (dq) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int f0 = 32 * fb + 8 * g + 4 * h;  // this lane holds features f0 .. f0+3 of its row
      __builtin_memcpy(kv[g], k + qk_row * C + f0, sizeof(kv[g]));
      __builtin_memcpy(qv[g], q + qk_row * C + f0, sizeof(qv[g]));
    }
  }
  const float d = diag[row];
  const float rq_i = rq[row], rk_i = rk[row];
  float l = 0.f, A = 0.f;
  {
    int s = 0;
    for (; s + 4 <= splits; s += 4) {
      float lv[4], av[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        lv[u] = lpart[(int64_t)(s + u) * npad + row];
        av[u] = apart[(int64_t)(s + u) * npad + row];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        l += lv[u];
        A += av[u];
      }
    }
    for (; s < splits; ++s) {
      l += lpart[(int64_t)s * npad + row];
      A += apart[(int64_t)s * npad + row];
    }
  }
  if (!dq) return;

  float o[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) o[i] = 0.f;
  const int64_t split_stride = (npad / 32) * FB * 16 * kWave;  // floats
  const f32x4* op0 = reinterpret_cast<const f32x4*>(opart + (tile32 * FB + fb) * 16 * kWave) + lane;
  int s0 = 0;
  for (; s0 + 4 <= splits; s0 += 4) {
    f32x4 v[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        v[u][g] = reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(op0) + (s0 + u) * split_stride)[g * kWave];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) o[4 * g + j] += v[u][g][j];
  }
  for (; s0 < splits; ++s0) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 v = reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(op0) + s0 * split_stride)[g * kWave];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[4 * g + j] += v[j];
    }
  }
  if (!live) return;
  const float inv_l = 1.f / l;
  const float gn = 2.f / (float)n;
  // below eps the norm is the constant eps and normalize() is linear: no projection
  const bool clamped = rq_i >= 1.f / kNormEps;
  const float dot = clamped ? 0.f : gn * (A * inv_l - d) / scale2;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int f0 = 32 * fb + 8 * g + 4 * h;
    T out[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float dqh = gn * (o[4 * g + j] * inv_l - to_f32(kv[g][j]) * rk_i);
      out[j] = from_f32<T>((dqh - to_f32(qv[g][j]) * rq_i * dot) * rq_i);
    }
    __builtin_memcpy(dq + row * C + f0, out, sizeof(out));
  }
}

template <typename T, int C>
int nce_run(const NceArgs& args, int pairs, int64_t n, float tau, const NceLayout& L, float* loss_out,
            hipStream_t stream) {
  const float scale2 = kNceLog2e / tau;
  const unsigned z = (unsigned)pairs;
  hipLaunchKernelGGL((nce_prep_kernel<T, C>), dim3((unsigned)(L.npad / kKTile), 1, z), dim3(kNceBlock), 0, stream, args,
                     n, L.npad, scale2);
  int rc = check_launch();
  if (rc) return rc;
  // see the kernel for the choice of the fastest grid index
  const bool qtile_major = (size_t)L.npad * C * 4 <= ((size_t)4 << 20);
  const dim3 main_grid = qtile_major ? dim3((unsigned)(L.npad / kQTile), (unsigned)L.splits, z)
                                     : dim3((unsigned)L.splits, (unsigned)(L.npad / kQTile), z);
  hipLaunchKernelGGL((nce_main_kernel<C>), main_grid, dim3(kNceBlock), 0, stream, args, n, L.npad, L.splits, scale2,
                     qtile_major ? 1 : 0);
  rc = check_launch();
  if (rc) return rc;
  const int64_t items = L.npad / 32 * (C / 32);  // a multiple of 4: npad is a multiple of 128
  hipLaunchKernelGGL((nce_combine_kernel<T, C>), dim3((unsigned)(items / 4 + 1), 1, z), dim3(kNceBlock), 0, stream,
                     args, n, L.npad, L.splits, scale2, 2.f * tau, loss_out);
  return check_launch();
}

template <typename T>
int nce_dispatch_c(const NceArgs& args, int pairs, int64_t n, int64_t c, float tau, const NceLayout& L,
                   float* loss_out, hipStream_t stream) {
  switch (c) {
    case 64: return nce_run<T, 64>(args, pairs, n, tau, L, loss_out, stream);
    case 128: return nce_run<T, 128>(args, pairs, n, tau, L, loss_out, stream);
    case 256: return nce_run<T, 256>(args, pairs, n, tau, L, loss_out, stream);
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
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
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
  ts::NceArgs args;
  for (int p = 0; p < 2; ++p) {
    const int src = p < pairs ? p : 0;  // an unused second slot mirrors the first
    char* wsp = ws + L.head_bytes + (size_t)src * L.pair_bytes;
    ts::NcePair& P = args.p[p];
    P.q = src ? q2 : q1;
    P.k = src ? k2 : k1;
    P.dq = src ? dq2 : dq1;
    P.rq = (float*)(wsp + L.off_rq);
    P.rk = (float*)(wsp + L.off_rk);
    P.diag = (float*)(wsp + L.off_diag);
    P.lpart = (float*)(wsp + L.off_lpart);
    P.apart = (float*)(wsp + L.off_apart);
    P.opart = (float*)(wsp + L.off_opart);
    P.kimg = (uint8_t*)(wsp + L.off_kimg);
    // fp32 and fp16 queries are rounded to a bf16 copy for the MFMA; bf16 ones are read in place
    P.qb = dtype != TS_BF16 ? (uint16_t*)(wsp + L.off_qb) : nullptr;
    P.qsrc = dtype != TS_BF16 ? P.qb : (const uint16_t*)P.q;
  }
  // loss = 2 tau / n * sum over all pairs' rows, written by the combine launch
  if (dtype == TS_F32) return ts::nce_dispatch_c<float>(args, pairs, n, c, tau, L, loss_out, st);
  if (dtype == TS_F16) return ts::nce_dispatch_c<ts::f16_t>(args, pairs, n, c, tau, L, loss_out, st);
  return ts::nce_dispatch_c<ts::bf16_t>(args, pairs, n, c, tau, L, loss_out, st);
}

}  // extern "C"
