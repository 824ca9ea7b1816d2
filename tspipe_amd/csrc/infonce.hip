// MoCo-v3 InfoNCE loss, forward and backward fused, on bf16 MFMA: the path
// for bf16 / fp16 embeddings of 64, 128 or 256 features at tau >= 0.03.  fp32
// embeddings, other widths and smaller temperatures run on the fp32 MFMA
// kernels of infonce_general.hip.
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
//     kernel; the queries feed the MFMA as they are (bf16 inputs in place,
//     fp16 inputs through a bf16 copy) and their 1/|q| is applied as an
//     fp32 factor after the contraction (logit_ij = <q_i, kh_j> * rq_i / tau).
//
// Kernels:
//   prep     per row: rq = 1/max(|q|,eps), rk, and the normalised key row
//            rounded to bf16 (row-major, zero rows up to a multiple of 128).
//   main     grid (q tile of 128 rows, key split); 8 wavefronts = 4 pairs, a
//            pair owning 32 q rows, two wavefronts on every SIMD.  Keys come
//            in stages of 64 (two tiles of 32), global memory -> LDS without
//            passing through registers, three buffers.  Per stage, wavefront
//            a of a pair computes S^T = Kh Q^T (MFMA 32x32x16) for tile a over
//            all features, P = 2^(S*scale - x_max) rounded to bf16, hands P to
//            its partner through LDS, and accumulates O^T += Kh^T P for ITS
//            HALF of the features over both tiles.  So a wavefront keeps 64
//            accumulator registers for O and 64 for its Q fragments and fits
//            in 256 registers.  The loop is software-pipelined with one
//            barrier per stage: the second product runs a stage behind the
//            first, and the exponentials of stage st are issued between the
//            MFMAs of the second product of stage st-1.  Kh^T operands are
//            read from the same row-major LDS tile as the Kh operands, with
//            the transposing LDS read of gfx950 (ds_read_b64_tr_b16).
//   combine  per 16 q rows: adds the key splits, forms dq; one more
//            workgroup adds up the loss from the split row sums.
//
// Accuracy: the row sum l is taken over the bf16-rounded P that the second
// product uses, so O / l is an exact convex combination of the rounded keys.
// The positive key's own term never enters O (the main kernel feeds P_ii to
// the second product as zero, while the row sum keeps it as it was rounded);
// the combine adds it with the fp32 kh_i.  The
// projection <qh, dqh> is formed from dqh itself.  The gradient then carries
// the bf16 rounding of the NEGATIVE keys only, weighted by their
// probabilities, also when P_ii -> 1.
//
// LDS tile: 64 key rows of C bf16, the 16-byte chunks of a row XOR-swizzled
// with a function of the row index chosen so that both operand reads are
// free of bank conflicts (nce_swz).
//
// MFMA 32x32x16 operand layout used throughout (lane l, half h = l/32):
//   A: row l%32, contraction slots 8h..8h+7;  B: column l%32, same slots;
//   D[i]: row (i%4) + 4h + 8(i/4), column l%32.
#include <atomic>
#include <type_traits>

#include "infonce_common.h"

// The LDS-DMA loads below set M0 from inline assembly and name it as
// clobbered, so that the compiler does not assume a value of its own survives
// them.  M0 is a register the compiler reserves, and it warns about any
// clobber of such a register; nothing here needs M0 preserved.
#pragma clang diagnostic ignored "-Winline-asm"

namespace ts {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int kQTile = 128;         // q rows per workgroup of the main kernel (32 per wavefront pair)
constexpr int kStageKeys = 64;      // keys per LDS stage (two tiles of 32)
constexpr int kNceBlock = 256;      // prep kernel
constexpr int kNceMainBlock = 512;  // main kernel: 8 wavefronts, two per SIMD

// defined in losses.hip
int launch_sum_scale(const float* v, int64_t n, float scale, float denom, float* out, hipStream_t stream);

// Workspace carve-up (all offsets multiples of 256 bytes): a small head, then
// one region per pair.
struct NceLayout {
  int64_t npad;
  int splits;
  size_t head_bytes;
  size_t off_rq, off_rk, off_pdiag, off_lpart, off_khat, off_qb, off_opart, pair_bytes;
};

// Key splits: enough workgroups for one per CU (a workgroup is 4 wavefronts,
// one per SIMD, each with its own software pipeline; its three stage buffers
// take most of a CU's LDS).
inline int nce_splits(int64_t npad, int n_pairs, int target) {
  const int64_t qtiles = npad / kQTile * n_pairs;
  const int64_t stages = npad / kStageKeys;
  int64_t s = (target + qtiles - 1) / qtiles;
  if (s > 16) s = 16;
  if (s > stages) s = stages;
  if (s < 1) s = 1;
  return (int)s;
}

inline NceLayout nce_layout(int64_t n, int64_t c, int n_pairs, int target) {
  NceLayout L;
  L.npad = nce_round_up(n > 0 ? n : 1, kQTile);
  L.splits = nce_splits(L.npad, n_pairs, target);
  L.head_bytes = 256;  // scratch for the empty-batch case
  size_t o = 0;
  L.off_rq = o;       o += nce_align(L.npad * 4);
  L.off_rk = o;       o += nce_align(L.npad * 4);
  L.off_pdiag = o;    o += nce_align(L.npad * 8);
  L.off_lpart = o;    o += nce_align((size_t)L.splits * L.npad * 4);
  L.off_khat = o;     o += nce_align((size_t)L.npad * c * 2);
  L.off_qb = o;       o += nce_align((size_t)L.npad * c * 2);  // used for fp16 inputs only
  L.off_opart = o;    o += nce_align((size_t)L.splits * L.npad * c * 4);
  L.pair_bytes = o;
  return L;
}

// ---------------------------------------------------------------------------
// prep: 16-byte row loads, a group of C/VEC lanes per row
// ---------------------------------------------------------------------------
template <typename T, int C>
struct NcePrep {
  static constexpr int VEC = 16 / sizeof(T);  // elements per 16-byte load
  static constexpr int LPR = C / VEC;         // lanes per row (8 .. 64)
  static constexpr int RPP = kWave / LPR;     // rows per wavefront pass
  static constexpr int ROWS = (4 * RPP > 16) ? 4 * RPP : 16;  // rows per workgroup (divides 64)
  static constexpr int NP = ROWS / (4 * RPP);                 // passes
};

template <typename T, int C>
__global__ __launch_bounds__(kNceBlock) void nce_prep_kernel(NceArgs args, int64_t n, int64_t npad) {
  const NcePair& pr = args.p[blockIdx.z];
  using P = NcePrep<T, C>;
  const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
  const int sub = lane / P::LPR, li = lane % P::LPR;  // row within the pass, lane within the row
  const int64_t row0 = (int64_t)blockIdx.x * P::ROWS;

  // the loads of all of this wavefront's rows go out before any is used
  u32x4 rawq[P::NP], rawk[P::NP];
#pragma unroll
  for (int pass = 0; pass < P::NP; ++pass) {
    const int64_t row = row0 + (pass * 4 + w) * P::RPP + sub;
    rawq[pass] = rawk[pass] = u32x4{0u, 0u, 0u, 0u};  // zero rows beyond n (0.0 in every dtype)
    if (row < n) {
      const NceRow rp = nce_row<T>(pr, row, C);
      rawq[pass] = *reinterpret_cast<const u32x4*>((const T*)rp.q + li * P::VEC);
      rawk[pass] = *reinterpret_cast<const u32x4*>((const T*)rp.k + li * P::VEC);
    }
  }
#pragma unroll
  for (int pass = 0; pass < P::NP; ++pass) {
    const int64_t row = row0 + (pass * 4 + w) * P::RPP + sub;
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
    uint16_t kbits[P::VEC], qbits[P::VEC];
#pragma unroll
    for (int e = 0; e < P::VEC; ++e) {
      kbits[e] = f32_to_bf16_bits(kv[e] * b);
      qbits[e] = f32_to_bf16_bits(qv[e]);
    }
    // VEC bf16 values: 16 bytes for the 2-byte input types, 8 for fp32
    __builtin_memcpy(pr.khat + row * C + li * P::VEC, kbits, sizeof(kbits));
    if (pr.qb) __builtin_memcpy(pr.qb + row * C + li * P::VEC, qbits, sizeof(qbits));
    if (li == 0) {
      pr.rq[row] = a;
      pr.rk[row] = b;
    }
  }
}

// ---------------------------------------------------------------------------
// main
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void nce_lds_void;
typedef __attribute__((address_space(1))) const void nce_glb_void;
typedef __attribute__((address_space(3))) s16x4 nce_lds_s16x4;

// XOR swizzle of the 16-byte chunk index of a row of the LDS tile.  Rows that
// differ in their low two bits get swizzles that differ in bits 2-3 and vice
// versa, which spreads over the banks both the 16 rows a quarter-wavefront
// reads at one chunk (first product) and the 4 rows x 4 chunks a
// quarter-wavefront reads in a transposing load (second product).
template <int CPR>
__device__ __forceinline__ int nce_swz(int row) {
  const int r = row & 15;
  return (((r & 3) << 2) | (r >> 2)) & (CPR - 1);
}

// HP: the partial O^T goes out as bf16 (inputs and gradient are 2-byte types
// anyway) instead of fp32, which halves the traffic between this kernel and
// the combine.
template <int C, bool HP>
__global__ __launch_bounds__(kNceMainBlock) void nce_main_kernel(NceArgs args, int64_t n, int64_t npad, int splits,
                                                                 float scale2 /* log2(e)/tau */, int qtile_major) {
  const NcePair& pr = args.p[blockIdx.z];
  constexpr int KK = C / 16;          // contraction steps of S^T
  constexpr int FBH = C / 64;         // 32-feature blocks of O^T per wavefront (half of the features)
  constexpr int CPR = C / 8;          // 16-byte chunks per key row
  constexpr int ROWB = C * 2;         // bytes per key row
  constexpr int STAGE = kStageKeys * ROWB;
  constexpr int NW = kNceMainBlock / kWave;
  constexpr int NU = STAGE / (NW * 1024);  // 1 KB fetches per wavefront and stage
  constexpr int KL = KK < 8 ? KK : 8;      // first-product chunk addresses kept in registers
  // Three stage buffers, stage st in buffer (st - s0) % 3: the one of the
  // first product, the one of the second product (a stage behind) and the one
  // being fetched.
  __shared__ __attribute__((aligned(1024))) uint8_t sm[3 * STAGE];
  // exchanged P, double-buffered by stage parity: [parity][pair][tile][step][lane * 16]
  __shared__ __attribute__((aligned(1024))) uint8_t xch[2][NW / 2][2][2][1024];
  constexpr int XPAR = (NW / 2) * 4096;  // bytes per parity
  __shared__ __attribute__((aligned(256))) uint8_t dump[NW * 256];  // written by the L2 prefetch, never read
  const int tid = threadIdx.x, lane = tid % kWave;
  const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int col = lane % 32, h = lane / 32;
  const int p = w >> 1, a = w & 1;
  // Workgroup ids are dealt round-robin to the 8 XCDs.  While all keys fit an
  // XCD's L2, the q tile is the fastest index: the key splits of a q tile run
  // on one XCD.  For more keys the split is the fastest index, so that an XCD
  // keeps seeing the same share of the keys.
  const int split = qtile_major ? blockIdx.y : blockIdx.x;
  const int64_t qtile = qtile_major ? blockIdx.x : blockIdx.y;
  const int64_t qrow = qtile * kQTile + p * 32 + col;  // the q row this lane is a column of

  const int stages = (int)(npad / kStageKeys);
  const int s0 = (int)((int64_t)stages * split / splits), s1 = (int)((int64_t)stages * (split + 1) / splits);

  // Every field of the pair that the prologue needs, requested in one go: one
  // scalar-load latency instead of one per use.
  const uint16_t* const khat_p = pr.khat;
  const uint16_t* const qb = pr.qb;
  const void* const q_single = pr.q;
  const float* const rq_p = pr.rq;
  const int n_pieces = pr.n_pieces;
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : : "s"(khat_p), "s"(qb), "s"(q_single), "s"(rq_p), "s"(n_pieces));
#else
  (void)khat_p, (void)qb, (void)q_single, (void)n_pieces;
#endif

  // Global -> LDS without passing through registers: lane L's 16 bytes land
  // at (LDS base) + 16 L, so the swizzle is applied on the global side: the
  // lane that fills slot (row, c') loads chunk c' ^ swz(row) of that row.
  uint32_t goff[NU];
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int slot = (w * NU + u) * kWave + lane;
    const int row = slot / CPR, cs = slot % CPR;
    goff[u] = (uint32_t)(row * ROWB + ((cs ^ nce_swz<CPR>(row)) << 4));
  }
  // one 1 KB piece of a stage (piece u of this wavefront's NU) into the buffer at byte offset `base`
  auto fetch_piece = [&](int st, int base, int u) {
    // Issued as assembly on purpose.  The compiler books an LDS-DMA load on
    // both memory counters and, while one is in flight, turns every wait for an
    // LDS read into a wait for ALL of them, which would undo the read-ahead of
    // the operand rings below.  Completion of these fetches is awaited
    // explicitly (vmcnt(0) in front of the stage barrier).  M0 carries the LDS
    // destination and is named as clobbered.
#if defined(__HIP_DEVICE_COMPILE__)
    const uint8_t* src = reinterpret_cast<const uint8_t*>(khat_p) + (int64_t)st * STAGE + goff[u];
    const uint32_t lds = (uint32_t)(uintptr_t)(nce_lds_void*)sm + (uint32_t)(base + (w * NU + u) * 1024);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(src), "s"(__builtin_amdgcn_readfirstlane(lds))
                 : "memory", "m0");
#endif
  };
  // The stage after the next is requested into this XCD's L2 (one word per
  // 128-byte line of this wavefront's share), so that the LDS fetch a stage
  // later finds it there: a fetch that has to go to memory does not always
  // land within one stage, and at the barrier every wavefront waits for the
  // slowest fetch of the eight.  The words go to an LDS area nobody reads: a
  // load into a register would write that register whenever it returns, long
  // after the compiler has given it to something else.  Issued after the
  // stage's fetches, so that vmcnt(1) awaits those and not this.
  auto l2_prefetch = [&](int st) {
#if defined(__HIP_DEVICE_COMPILE__)
    if (lane < 8 * NU) {
      const uint8_t* src = reinterpret_cast<const uint8_t*>(khat_p) + (int64_t)st * STAGE + (w * NU * 8 + lane) * 128;
      const uint32_t lds = (uint32_t)(uintptr_t)(nce_lds_void*)dump + (uint32_t)(w * 256);
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
                   :
                   : "v"(src), "s"(__builtin_amdgcn_readfirstlane(lds))
                   : "memory", "m0");
    }
#else
    (void)st, (void)dump;
#endif
  };
  if (s0 < s1) {
#pragma unroll
    for (int u = 0; u < NU; ++u) fetch_piece(s0, 0, u);
    l2_prefetch(s0 + 1 < s1 ? s0 + 1 : s1 - 1);
  }

  const float rq_i = (qrow < n) ? rq_p[qrow] : 0.f;  // on its way while the tiles are fetched
  const float sc_i = rq_i * scale2;

  // Q fragments: B operand of S^T, resident for the whole kernel.  The q tile
  // (kQTile rows, exactly two stage buffers) comes in through LDS with the
  // same swizzled, coalesced fetch as the keys; read straight from global
  // memory, a fragment load would touch 64 different cache lines.
  // Rows beyond the batch fetch the last row instead; their fragments are
  // zeroed below.  One decision up front (a single matrix, or row blocks), so
  // that the pair's fields are read once and the eight fetches go out back to
  // back.
#if defined(__HIP_DEVICE_COMPILE__)
  {
    const uint32_t lds0 = (uint32_t)(uintptr_t)(nce_lds_void*)sm + (uint32_t)(STAGE + w * 2 * NU * 1024);
    auto fetch_q = [&](auto&& row_ptr, uint32_t lds_base) {
      const uint8_t* qsrc[2 * NU];
#pragma unroll
      for (int u = 0; u < 2 * NU; ++u) {
        const int slot = (w * 2 * NU + u) * kWave + lane;
        const int row = slot / CPR, cs = slot % CPR;
        int64_t grow = qtile * kQTile + row;
        grow = grow < n ? grow : n - 1;
        qsrc[u] = reinterpret_cast<const uint8_t*>(row_ptr(grow)) + ((cs ^ nce_swz<CPR>(row)) << 4);
      }
#pragma unroll
      for (int u = 0; u < 2 * NU; ++u) {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :
                     : "v"(qsrc[u]), "s"(__builtin_amdgcn_readfirstlane(lds_base + u * 1024))
                     : "memory", "m0");
      }
    };
    if (qb != nullptr || n_pieces == 0) {
      const uint16_t* base = qb ? qb : (const uint16_t*)q_single;
      fetch_q([&](int64_t grow) { return base + grow * C; }, lds0);
    } else {
      fetch_q([&](int64_t grow) { return (const uint16_t*)nce_row<bf16_t>(pr, grow, C).q; }, lds0);
    }
  }
#endif
  __builtin_amdgcn_s_waitcnt(0x0070);
  __builtin_amdgcn_s_barrier();  // the q tile and stage s0 are in LDS
  bf16x8 qf[KK];
  {
    const int row = p * 32 + col;
    const int sw = nce_swz<CPR>(row);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      u32x4 raw = *reinterpret_cast<const u32x4*>(sm + STAGE + row * ROWB + (((2 * kk + h) ^ sw) << 4));
      if (qrow >= n) raw = u32x4{0u, 0u, 0u, 0u};  // rows beyond the batch were not fetched
      __builtin_memcpy(&qf[kk], &raw, 16);
    }
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // the fragments have left LDS ...
  __builtin_amdgcn_s_barrier();        // ... in every wavefront: the two buffers may be fetched into

  // LDS byte offsets of this lane's operand reads within a stage (the parts
  // that depend on a compile-time index only through an addition are left to
  // the instruction's immediate offset; the buffer's base is added per stage).
  // first product, A operand: key row 32a + col, chunk 2kk + h
  uint32_t ak[KL];
  {
    const int row = 32 * a + col;
    const int sw = nce_swz<CPR>(row);
#pragma unroll
    for (int kl = 0; kl < KL; ++kl) ak[kl] = (uint32_t)(row * ROWB + (((2 * kl + h) ^ sw) << 4));
  }
  // second product, A operand through the transposing read: within a group of
  // 16 lanes, lane s supplies the address of 4 features of one key row and
  // receives one feature of 4 key rows.  Group g = lane / 16 covers features
  // 16 (g % 2) .. +15 of a 32-feature block and the key slots of half g / 2.
  uint32_t at[FBH][2];
  {
    const int g = lane >> 4, s = lane & 15;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int row = 8 * r + 4 * (g >> 1) + (s >> 2);
      const int sw = nce_swz<CPR>(row);
#pragma unroll
      for (int fbl = 0; fbl < FBH; ++fbl) {
        const int chunk = 4 * (a * FBH + fbl) + 2 * (g & 1) + ((s & 3) >> 1);
        at[fbl][r] = (uint32_t)(row * ROWB + ((chunk ^ sw) << 4) + 8 * (s & 1));
      }
    }
  }

  f32x16 oacc[FBH];
#pragma unroll
  for (int fb = 0; fb < FBH; ++fb)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[fb][i] = 0.f;
  float lsum = 0.f;                      // sum_j of the bf16-rounded P_ij over this wavefront's tiles
  float pd_exact = 0.f, pd_round = 0.f;  // P_ii before and after the rounding (set by the lane that meets it)
  const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
  // the lane of column col that holds key `col` of a diagonal tile: D register i*, half h*
  const int hstar = (col >> 2) & 1, istar = (col & 3) + 4 * (col >> 3);
  // the pair's own keys are tile p of the q tile's four: stage 2 qtile + p/2, its tile p%2
  const int diag_stage = (int)(2 * qtile) + (p >> 1);
  const bool diag_wave = a == (p & 1);

  // Software pipeline, one barrier per stage.  In stage st a wavefront issues
  //   16 MFMAs of S^T(st)                     (+ the fetches of stage st+1),
  //   16 MFMAs of O^T += Kh^T(st-1) P(st-1)   with the soft-max of S^T(st)
  //                                           between them on the vector unit,
  // then writes P(st) for its partner and meets the others at the barrier.  A
  // SIMD holds two wavefronts of the workgroup, so the vector work of one runs
  // under the MFMAs of the other.
  //
  // Operand fragments are read from LDS four MFMAs ahead of their use, into a
  // ring of four register sets, and the read-ahead runs across the phases: the
  // first operands of the second product are requested during the last steps
  // of the first.  The order is pinned with scheduling barriers, because left
  // to itself the compiler reads every fragment right in front of its MFMA
  // and the LDS latency is paid at every step.  (Holding the last MFMAs of the
  // second product back over the barrier, to cover the first reads of the next
  // stage, was measured: no gain.)
  constexpr int RING = 4;
  constexpr int NSTEP = 4 * FBH;  // MFMAs of the second product per stage (== KK), which also carry the soft-max
  static_assert(NSTEP == KK && NSTEP <= 16, "feature width");
  const uint32_t xlane = (uint32_t)(p * 4096 + lane * 16);
  uint8_t* const xch0 = &xch[0][0][0][0][0];
  // Second product: O^T[f][q] += sum_key Kh^T[f][key] P[key][q] over both tiles
  // of a stage, for this wavefront's half of the features; contraction slot
  // 8h + 4r + j of step T is key 16T + 8r + 4h + j on both operands.
  // step s: key step T = s / FBH (16 keys), feature block s % FBH.
  auto read_t = [&](const uint32_t (&atc)[FBH][2], int step) {
    const int T = step / FBH, fbl = step % FBH;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((nce_lds_s16x4*)(sm + atc[fbl][0] + T * 16 * ROWB));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((nce_lds_s16x4*)(sm + atc[fbl][1] + T * 16 * ROWB));
    bf16x8 v;
    __builtin_memcpy(&v, &lo, 8);
    __builtin_memcpy(reinterpret_cast<char*>(&v) + 8, &hi, 8);
    return v;
  };
  auto read_p = [&](int parity, int T) {
    const u32x4 praw = *reinterpret_cast<const u32x4*>(xch0 + parity * XPAR + xlane + T * 1024);
    bf16x8 v;
    __builtin_memcpy(&v, &praw, 16);
    return v;
  };
  // MODE 0: the split's first stage (no second product yet), 1: any later stage.
  // cur / prev / nxt: byte offsets of the buffers of stages st, st-1, st+1.
  auto one_stage = [&](int st, int cur, int prev, int nxt, auto mode_tag) {
    constexpr int MODE = decltype(mode_tag)::value;
    uint32_t akc[KL];
#pragma unroll
    for (int kl = 0; kl < KL; ++kl) akc[kl] = ak[kl] + (uint32_t)cur;
    uint32_t atc[FBH][2];
#pragma unroll
    for (int fbl = 0; fbl < FBH; ++fbl) {
      atc[fbl][0] = at[fbl][0] + (uint32_t)prev;
      atc[fbl][1] = at[fbl][1] + (uint32_t)prev;
    }
    auto read_k = [&](int kk) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(sm + akc[kk % KL] + (kk / KL) * (KL * 32));
      bf16x8 v;
      __builtin_memcpy(&v, &raw, 16);
      return v;
    };
    // near the end the fetch repeats the last stage into the idle buffer (no branch)
    const int st_next = st + 1 < s1 ? st + 1 : s1 - 1;
    const int par_prev = (st - 1) & 1;

    bf16x8 kr[RING];
#pragma unroll
    for (int i = 0; i < RING; ++i) kr[i] = read_k(i);
    __builtin_amdgcn_sched_barrier(0);

    // S^T[key][q] = sum_f Kh[key][f] Q[q][f] for tile a of the stage; the
    // next stage's fetches are issued between the MFMAs, into the buffer that
    // held stage st-2 (every wavefront finished with it before the barrier
    // that ended stage st-1)
    f32x16 sacc;
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
    bf16x8 pbT[4], tr[RING];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kr[kk % RING], qf[kk], sacc, 0, 0, 0);
      if (kk + RING < KK) kr[kk % RING] = read_k(kk + RING);
      if (MODE >= 1 && kk >= KK - RING) {  // first operands of the second product
        const int j = kk - (KK - RING);
        if (j < 2) {
          pbT[2 * j] = read_p(par_prev, 2 * j);
          pbT[2 * j + 1] = read_p(par_prev, 2 * j + 1);
        }
        tr[j] = read_t(atc, j);
      }
      if (kk < NU) fetch_piece(st_next, nxt, kk);
      if (kk == NU) l2_prefetch(st + 2 < s1 ? st + 2 : s1 - 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    // P = 2^(S * rq_i * log2e/tau - x_max), rounded to bf16; keys this lane
    // holds: key(i) = (i%4) + 4h + 8(i/4).  The row sum is taken over the
    // rounded values (v_dot2 of the packed pairs with ones).
    float pv[16];
    float pe = 0.f;
    bf16x8 pb[2];
    auto softmax_elems = [&](int i0, int i1) {
#pragma unroll
      for (int i = i0; i < i1; ++i) {
        pv[i] = fast_exp2(fmaf(sacc[i], sc_i, -scale2));
        pe = (i == istar) ? pv[i] : pe;
        if (i & 1) {
          const bf16x2 pk = {(__bf16)pv[i - 1], (__bf16)pv[i]};
          lsum = __builtin_amdgcn_fdot2_f32_bf16(pk, ones, lsum, false);
          pb[i / 8][(i - 1) % 8] = pk[0];
          pb[i / 8][i % 8] = pk[1];
        }
      }
    };
    if (MODE == 0) {
      softmax_elems(0, 16);
    } else {
#pragma unroll
      for (int step = 0; step < NSTEP; ++step) {
        oacc[step % FBH] =
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr[step % RING], pbT[step / FBH], oacc[step % FBH], 0, 0, 0);
        if (step + RING < NSTEP) tr[step % RING] = read_t(atc, step + RING);
        softmax_elems(16 * step / NSTEP, 16 * (step + 1) / NSTEP);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (st == diag_stage && diag_wave) {  // the tile that holds this pair's own keys (uniform)
      // The positive key's own term leaves the second product here: P~_ii stays
      // in the row sum above but goes to the MFMA as zero, so O^T is the
      // negatives' sum and the combine adds (1 - P~_ii / l~) kh_i in fp32.
      if (h == hstar) {
        pd_exact = pe;
        pd_round = (float)(__bf16)pe;
      }
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (i == istar && h == hstar) pb[i / 8][i % 8] = (__bf16)0.0f;
    }
    // hand this tile's P to the partner (and to this wavefront's own second product)
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      u32x4 raw;
      __builtin_memcpy(&raw, &pb[t2], 16);
      *reinterpret_cast<u32x4*>(xch0 + (st & 1) * XPAR + xlane + a * 2048 + t2 * 1024) = raw;
    }
    // After this barrier: P(st) is visible, stage st+1 is complete in LDS (every
    // wavefront waited for its own pieces) and everybody has finished reading
    // stage st-1 and P(st-1).
    __builtin_amdgcn_s_waitcnt(0x0071);  // vmcnt(1): all but the L2 prefetch, which came last; lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
  };

  if (s0 < s1) {
    int cur = 0, prev = 2 * STAGE, nxt = STAGE;
    auto rotate = [&]() {
      const int t = prev;
      prev = cur;
      cur = nxt;
      nxt = t;
    };
    one_stage(s0, cur, prev, nxt, std::integral_constant<int, 0>{});
    for (int st = s0 + 1; st < s1; ++st) {
      rotate();
      one_stage(st, cur, prev, nxt, std::integral_constant<int, 1>{});
    }
    // the second product of the last stage
    {
      uint32_t atc[FBH][2];
#pragma unroll
      for (int fbl = 0; fbl < FBH; ++fbl) {
        atc[fbl][0] = at[fbl][0] + (uint32_t)cur;
        atc[fbl][1] = at[fbl][1] + (uint32_t)cur;
      }
      const int parity = (s1 - 1) & 1;
      bf16x8 pbT[4], tr[RING];
#pragma unroll
      for (int T = 0; T < 4; ++T) pbT[T] = read_p(parity, T);
#pragma unroll
      for (int i = 0; i < RING; ++i) tr[i] = read_t(atc, i);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int step = 0; step < NSTEP; ++step) {
        oacc[step % FBH] =
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(tr[step % RING], pbT[step / FBH], oacc[step % FBH], 0, 0, 0);
        if (step + RING < NSTEP) tr[step % RING] = read_t(atc, step + RING);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // The last L2 prefetch writes into this workgroup's LDS; it must have landed
  // before the LDS can be handed to another workgroup.
  __builtin_amdgcn_s_waitcnt(0x0f70);

  // Padded keys (zero rows of Kh) took part in the row sums with the same
  // term for every row, the rounded 2^(0 - x_max); take this lane's share out.
  {
    int cnt = 0;
    const int st_pad = (int)(n / kStageKeys);
    for (int st = (s0 > st_pad ? s0 : st_pad); st < s1; ++st)
#pragma unroll
      for (int i = 0; i < 16; ++i) cnt += ((int64_t)st * kStageKeys + 32 * a + 4 * h + 8 * (i / 4) + (i % 4) >= n) ? 1 : 0;
    const float c0 = (float)(__bf16)fast_exp2(fmaf(0.f, sc_i, -scale2));
    lsum -= (float)cnt * c0;
  }

  // row sums: the two halves of a lane pair, then the two wavefronts of the pair (through LDS)
  const bool has_diag = diag_stage >= s0 && diag_stage < s1;  // this split met the pair's own keys (uniform)
  float ltot = lsum + __shfl_xor(lsum, 32, kWave);
  __syncthreads();  // everybody is done with xch
  float* lx = reinterpret_cast<float*>(&xch[0][0][0][0][0]);
  if (a == 1 && h == 0) lx[p * 32 + col] = ltot;
  __syncthreads();
  if (a == 0 && h == 0) {
    ltot += lx[p * 32 + col];
    pr.lpart[(int64_t)split * npad + qrow] = ltot;
  }
  if (has_diag && diag_wave && h == hstar) {
    const f32x2 v = {pd_exact, pd_round};
    *reinterpret_cast<f32x2*>(pr.pdiag + 2 * qrow) = v;
  }
  // partial O^T in register-native order, [split][tile of 32 q rows][feature half a][fb] and then
  //   fp32: [i/4][lane][i%4]      (16 bytes per lane and store)
  //   bf16: [i/8][lane][i%8]      (16 bytes per lane and store)
  const int64_t tile32 = qtile * (kQTile / 32) + p;
  const int64_t blk = (((int64_t)split * (npad / 32) + tile32) * 2 + a) * FBH;  // 32-feature blocks in front
  if (HP) {
    u32x4* op = reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(pr.opart) + blk * 16 * kWave);
#pragma unroll
    for (int fb = 0; fb < FBH; ++fb)
#pragma unroll
      for (int g2 = 0; g2 < 2; ++g2) {
        bf16x8 v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (__bf16)oacc[fb][8 * g2 + e];
        u32x4 raw;
        __builtin_memcpy(&raw, &v, 16);
        op[(fb * 2 + g2) * kWave + lane] = raw;
      }
  } else {
    f32x4* op = reinterpret_cast<f32x4*>(pr.opart + blk * 16 * kWave);
#pragma unroll
    for (int fb = 0; fb < FBH; ++fb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 v = {oacc[fb][4 * g], oacc[fb][4 * g + 1], oacc[fb][4 * g + 2], oacc[fb][4 * g + 3]};
        op[(fb * 4 + g) * kWave + lane] = v;
      }
  }
}

// ---------------------------------------------------------------------------
// combine: one workgroup per 16 q rows, one wavefront per 32-feature block.
// Lane (row = lane % 16, h, g2) of wavefront fb holds features
// 32 fb + 8 g + 4 h + j for g = 2 g2, 2 g2 + 1 and j = 0..3, the order the
// partial O^T was stored in.  With O'_i the negatives' sum (the main kernel
// kept the positive key's term out):
//   dqh_i = (2/N) [ O'_i / l~_i  -  (1 - P~_ii / l~_i) kh_i ]
// (~: rounded to bf16 as the MFMA saw it; kh_i: fp32), then the projection
// with <qh_i, dqh_i>, summed over the row through LDS.
// ---------------------------------------------------------------------------
// The scalar loss, by one workgroup straight from the split row sums:
//   loss = loss_scale / n * sum over pairs and rows of ln( l_i / P_ii ),
//   l_i = (l~_i - P~_ii) + P_ii  (the positive term unrounded).
// Re-deriving l_i here instead of reading the other workgroups' results keeps
// the reduction inside this launch; the order of every addition is fixed.
// QN x 4 rows per thread and trip, all loads of a trip issued before the first
// use: the workgroup walks the whole batch alone, so its time is the number
// of trips times the memory latency.  SC: splits requested in one go, as in the
// combine kernel (QN shrinks as SC grows; the registers are what bounds both).
template <int NT, int SC>
__device__ __forceinline__ void nce_loss_block(const NceArgs& args, int pairs, int64_t n, int64_t npad, int splits,
                                               float loss_scale, float* __restrict__ loss_out) {
  __shared__ float red[NT / kWave];
  const int tid = threadIdx.x;
  constexpr int QN = SC == 2 ? 4 : (SC == 4 ? 2 : 1);
  float acc = 0.f;
  for (int p = 0; p < pairs; ++p) {
    const float* __restrict__ lpart = args.p[p].lpart;
    const float* __restrict__ pdiag = args.p[p].pdiag;
    const int64_t nquad = npad / 4;
    for (int64_t q0 = tid; q0 < nquad; q0 += (int64_t)NT * QN) {
      f32x4 d0[QN], d1[QN], l[QN];
#pragma unroll
      for (int u = 0; u < QN; ++u) {
        const int64_t quad = q0 + (int64_t)u * NT < nquad ? q0 + (int64_t)u * NT : q0;  // beyond the end: re-read, dropped below
        d0[u] = *reinterpret_cast<const f32x4*>(pdiag + 8 * quad);      // rows 4q, 4q+1: exact, rounded
        d1[u] = *reinterpret_cast<const f32x4*>(pdiag + 8 * quad + 4);  // rows 4q+2, 4q+3
        l[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
      for (int s0 = 0; s0 < splits; s0 += SC) {
        f32x4 v[QN][SC];
#pragma unroll
        for (int u = 0; u < QN; ++u) {
          const int64_t quad = q0 + (int64_t)u * NT < nquad ? q0 + (int64_t)u * NT : q0;
#pragma unroll
          for (int c = 0; c < SC; ++c) {
            const int sp = s0 + c < splits ? s0 + c : s0;
            v[u][c] = *reinterpret_cast<const f32x4*>(lpart + (int64_t)sp * npad + 4 * quad);
          }
        }
#pragma unroll
        for (int u = 0; u < QN; ++u)
#pragma unroll
          for (int c = 0; c < SC; ++c) l[u] += v[u][c] * (s0 + c < splits ? 1.f : 0.f);
      }
#pragma unroll
      for (int u = 0; u < QN; ++u) {
        const int64_t quad = q0 + (int64_t)u * NT;
        const float pe[4] = {d0[u][0], d0[u][2], d1[u][0], d1[u][2]}, pr[4] = {d0[u][1], d0[u][3], d1[u][1], d1[u][3]};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float t = kNceLn2 * (log2f((l[u][j] - pr[j]) + pe[j]) - log2f(pe[j]));
          acc += (quad < nquad && 4 * quad + j < n) ? t : 0.f;
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
    for (int w = 0; w < NT / kWave; ++w) total += red[w];
    *loss_out = total * loss_scale / (float)n;
  }
}

// SC: key splits whose partial sums a thread requests in one go (2, 4 or 8,
// the smallest that covers the launch's split count, more come in further
// rounds); slots beyond the split count re-read a valid split and are dropped.
template <typename T, int C, bool HP, int SC>
__global__ __launch_bounds__(2 * C) void nce_combine_kernel(NceArgs args, int64_t n, int64_t npad, int splits,
                                                            float loss_scale, float* __restrict__ loss_out,
                                                            int xcd_map) {
  constexpr int NW = C / 32;  // wavefronts: one per 32-feature block
  constexpr int FBH = C / 64;
  // The grid is the 16-row units, then 8 more workgroups of which the first
  // computes the loss (for the first pair only) and the others have nothing to do.
  const int64_t units = npad / 16;
  if (blockIdx.x >= units) {
    if (blockIdx.x == units && blockIdx.z == 0)
      nce_loss_block<2 * C, SC>(args, (int)gridDim.z, n, npad, splits, loss_scale, loss_out);
    return;
  }
  // Workgroup ids are dealt round-robin to the 8 XCDs and the grid's width is
  // a multiple of 8.  With xcd_map, the main kernel ran all key splits of q
  // tile t on XCD t % 8; a unit is taken by a workgroup of that XCD, which
  // finds the partial sums in its own L2.
  int64_t unit = blockIdx.x;
  if (xcd_map) {
    const int64_t x = blockIdx.x % 8, j = blockIdx.x / 8;
    constexpr int UPT = kQTile / 16;  // units per q tile
    unit = (x + 8 * (j / UPT)) * UPT + j % UPT;
  }
  const NcePair& pr = args.p[blockIdx.z];
  __shared__ float dots[NW][16];
  const int lane = threadIdx.x % kWave, fb = threadIdx.x / kWave;
  const int col16 = lane & 15, h = (lane >> 4) & 1, g2 = lane >> 5;
  const int64_t tile32 = unit >> 1;
  const int half = (int)(unit & 1);
  const int64_t row = unit * 16 + col16;
  const bool live = row < n;
  const int a = fb / FBH, fbl = fb % FBH;
  const int slot = h * 32 + half * 16 + col16;  // the main kernel's lane that held this row and feature group

  // Bound by memory latency, not arithmetic: every load is issued before the
  // first use of any of them (up to 8 splits; more come in further rounds).
  const int64_t qk_row = live ? row : 0;  // padded rows read row 0 and discard it
  const NceRow rp = nce_row<T>(pr, qk_row, C);
  T kv[2][4], qv[2][4];
#pragma unroll
  for (int gg = 0; gg < 2; ++gg) {
    const int f0 = 32 * fb + 8 * (2 * g2 + gg) + 4 * h;  // this lane holds features f0 .. f0+3 of its row
    __builtin_memcpy(kv[gg], (const T*)rp.k + f0, sizeof(kv[gg]));
    __builtin_memcpy(qv[gg], (const T*)rp.q + f0, sizeof(qv[gg]));
  }
  const f32x2 pd = *reinterpret_cast<const f32x2*>(pr.pdiag + 2 * row);
  const float rq_i = pr.rq[row], rk_i = pr.rk[row];
  float o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = 0.f;
  float l = 0.f;
  const int64_t blk = (tile32 * 2 + a) * FBH + fbl;                // 32-feature blocks in front, within a split
  const int64_t split_blocks = (npad / 32) * 2 * FBH;              // 32-feature blocks per split
  for (int s0 = 0; s0 < splits; s0 += SC) {
    float lv[SC];
    f32x4 vf[SC][2];
    u32x4 vh[SC];
#pragma unroll
    for (int u = 0; u < SC; ++u) {
      const int sp = s0 + u < splits ? s0 + u : s0;  // a split beyond the end re-reads a valid one and is dropped
      lv[u] = pr.lpart[(int64_t)sp * npad + row];
      const int64_t b = (int64_t)sp * split_blocks + blk;
      if (HP) {
        vh[u] = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(pr.opart) + b * 16 * kWave)[g2 * kWave + slot];
      } else {
        const f32x4* src = reinterpret_cast<const f32x4*>(pr.opart + b * 16 * kWave);
        vf[u][0] = src[(2 * g2) * kWave + slot];
        vf[u][1] = src[(2 * g2 + 1) * kWave + slot];
      }
    }
#pragma unroll
    for (int u = 0; u < SC; ++u) {
      if (s0 + u >= splits) continue;
      l += lv[u];
      if (HP) {
        uint16_t hb[8];
        __builtin_memcpy(hb, &vh[u], 16);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] += bf16_bits_to_f32(hb[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] += vf[u][e / 4][e % 4];
      }
    }
  }
  const float inv_l = 1.f / l;
  const float gn = 2.f / (float)n;
  const float w_neg = (l - pd[1]) * inv_l;  // 1 - P~_ii / l~
  float dqh[8], qh[8];
  float dot = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    dqh[e] = gn * (o[e] * inv_l - w_neg * (to_f32(kv[e / 4][e % 4]) * rk_i));
    qh[e] = to_f32(qv[e / 4][e % 4]) * rq_i;
    dot = fmaf(qh[e], dqh[e], dot);
  }
  dot += __shfl_xor(dot, 16, kWave);
  dot += __shfl_xor(dot, 32, kWave);
  if (lane < 16) dots[fb][col16] = dot;
  __syncthreads();
  if (!live || !rp.dq) return;
  float total = 0.f;
#pragma unroll
  for (int x = 0; x < NW; ++x) total += dots[x][col16];
  // below eps the norm is the constant eps and normalize() is linear: no projection
  if (rq_i >= 1.f / kNormEps) total = 0.f;
#pragma unroll
  for (int gg = 0; gg < 2; ++gg) {
    const int f0 = 32 * fb + 8 * (2 * g2 + gg) + 4 * h;
    T out[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = from_f32<T>((dqh[4 * gg + j] - qh[4 * gg + j] * total) * rq_i);
    __builtin_memcpy((T*)rp.dq + f0, out, sizeof(out));
  }
}

template <typename T, int C>
int nce_run(const NceArgs& args, int pairs, int64_t n, float tau, const NceLayout& L, float* loss_out,
            hipStream_t stream) {
  const float scale2 = kNceLog2e / tau;
  const unsigned z = (unsigned)pairs;
  using P = NcePrep<T, C>;
  hipLaunchKernelGGL((nce_prep_kernel<T, C>), dim3((unsigned)(L.npad / P::ROWS), 1, z), dim3(kNceBlock), 0, stream, args,
                     n, L.npad);
  int rc = check_launch();
  if (rc) return rc;
  // see the kernel for the choice of the fastest grid index
  const bool qtile_major = (size_t)L.npad * C * 2 <= ((size_t)4 << 20);
  const dim3 main_grid = qtile_major ? dim3((unsigned)(L.npad / kQTile), (unsigned)L.splits, z)
                                     : dim3((unsigned)L.splits, (unsigned)(L.npad / kQTile), z);
  // the 2-byte types, whose gradient is rounded to 2^-9 anyway, keep bf16 partial sums
  constexpr bool HP = sizeof(T) == 2;
  hipLaunchKernelGGL((nce_main_kernel<C, HP>), main_grid, dim3(kNceMainBlock), 0, stream, args, n, L.npad, L.splits, scale2,
                     qtile_major ? 1 : 0);
  rc = check_launch();
  if (rc) return rc;
  const int xcd_map = qtile_major && (L.npad / kQTile) % 8 == 0 ? 1 : 0;
  const dim3 cgrid((unsigned)(L.npad / 16 + 8), 1, z);
  if (L.splits <= 2)
    hipLaunchKernelGGL((nce_combine_kernel<T, C, HP, 2>), cgrid, dim3(2 * C), 0, stream, args, n, L.npad, L.splits,
                       2.f * tau, loss_out, xcd_map);
  else if (L.splits <= 4)
    hipLaunchKernelGGL((nce_combine_kernel<T, C, HP, 4>), cgrid, dim3(2 * C), 0, stream, args, n, L.npad, L.splits,
                       2.f * tau, loss_out, xcd_map);
  else
    hipLaunchKernelGGL((nce_combine_kernel<T, C, HP, 8>), cgrid, dim3(2 * C), 0, stream, args, n, L.npad, L.splits,
                       2.f * tau, loss_out, xcd_map);
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

// Fills the per-pair workspace pointers and launches.
int nce_launch(NceArgs& args, int pairs, int64_t n, int64_t c, float tau, void* workspace, float* loss_out,
               int dtype, hipStream_t st) {
  const NceLayout L = nce_layout(n, c, pairs, nce_workgroup_target());
  char* ws = (char*)workspace;
  for (int p = 0; p < 2; ++p) {
    const int src = p < pairs ? p : 0;  // an unused second slot mirrors the first
    if (p >= pairs) args.p[p] = args.p[0];
    char* wsp = ws + L.head_bytes + (size_t)src * L.pair_bytes;
    NcePair& P = args.p[p];
    P.rq = (float*)(wsp + L.off_rq);
    P.rk = (float*)(wsp + L.off_rk);
    P.pdiag = (float*)(wsp + L.off_pdiag);
    P.lpart = (float*)(wsp + L.off_lpart);
    P.opart = (float*)(wsp + L.off_opart);
    P.khat = (uint16_t*)(wsp + L.off_khat);
    // fp16 queries are rounded to a bf16 copy for the MFMA; bf16 ones are read in place
    P.qb = dtype != TS_BF16 ? (uint16_t*)(wsp + L.off_qb) : nullptr;
  }
  // loss = 2 tau / n * sum over all pairs' rows, written by the combine launch
  if (dtype == TS_F32) return TS_ERR_ARG;  // fp32 embeddings never take this path (nce_bf16_path)
  if (dtype == TS_F16) return nce_dispatch_c<f16_t>(args, pairs, n, c, tau, L, loss_out, st);
  return nce_dispatch_c<bf16_t>(args, pairs, n, c, tau, L, loss_out, st);
}

inline void nce_clear_pieces(NcePair& P) {
  P.q = P.k = nullptr;
  P.dq = nullptr;
  P.rq = P.rk = P.pdiag = P.lpart = P.opart = P.stat = nullptr;
  P.khat = P.qb = nullptr;
  P.n_pieces = 0;
  for (int i = 0; i < kNceMaxPieces; ++i) {
    P.row0[i] = 0;
    P.qp[i] = P.kp[i] = nullptr;
    P.dqp[i] = nullptr;
  }
}

// The bf16-MFMA path takes 2-byte inputs of width 64 / 128 / 256 at
// temperatures its fixed soft-max reference point can represent
// (2^(-2 log2(e)/tau) must stay a normal fp32); everything else -- fp32 inputs,
// other widths, smaller temperatures -- goes to the fp32-MFMA path.
static std::atomic<int> g_nce_fp32_arithmetic{0};

inline bool nce_bf16_path(int64_t c, float tau, int dtype) {
  if (g_nce_fp32_arithmetic.load(std::memory_order_relaxed)) return false;
  return dtype != TS_F32 && (c == 64 || c == 128 || c == 256) && tau >= 0.03f;
}

static std::atomic<int> g_nce_workgroup_target{kNceMaxWorkgroupTarget};
int nce_workgroup_target() { return g_nce_workgroup_target.load(std::memory_order_relaxed); }

}  // namespace ts

extern "C" {

int ts_infonce_set_workgroup_target(int workgroups) {
  if (workgroups <= 0 || workgroups > ts::kNceMaxWorkgroupTarget) workgroups = ts::kNceMaxWorkgroupTarget;
  return ts::g_nce_workgroup_target.exchange(workgroups, std::memory_order_relaxed);
}

int ts_infonce_set_fp32_arithmetic(int on) {
  return ts::g_nce_fp32_arithmetic.exchange(on ? 1 : 0, std::memory_order_relaxed);
}

size_t ts_infonce_workspace_bytes(int64_t n, int64_t c, int n_pairs) {
  if (n < 0 || c <= 0 || c > 512 || n_pairs < 1 || n_pairs > 2) return 0;
  // dtype and temperature decide the path at call time: room for either
  size_t bytes = ts::nce_general_workspace_bytes(n, c, n_pairs);
  if (c == 64 || c == 128 || c == 256) {
    const ts::NceLayout L = ts::nce_layout(n, c, n_pairs, ts::kNceMaxWorkgroupTarget);
    const size_t b16 = L.head_bytes + L.pair_bytes * (size_t)n_pairs;
    if (b16 > bytes) bytes = b16;
  }
  return bytes;
}

int ts_infonce_fwd_bwd(const void* q1, const void* k1, const void* q2, const void* k2, int64_t n, int64_t c,
                       float tau, void* workspace, float* loss_out, void* dq1, void* dq2, int dtype,
                       ts_stream_t stream) {
  if (!loss_out || (n > 0 && (!q1 || !k1 || !workspace))) return TS_ERR_ARG;
  if ((q2 == nullptr) != (k2 == nullptr)) return TS_ERR_ARG;
  if (n < 0 || !(tau > 0.f) || c < 1) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (c > 512 || n > (1 << 24)) return TS_ERR_RANGE;
  if ((uintptr_t)workspace & 255u) return TS_ERR_ALIGN;
  const uintptr_t ptr_bits = (uintptr_t)q1 | (uintptr_t)k1 | (uintptr_t)q2 | (uintptr_t)k2 | (uintptr_t)dq1 | (uintptr_t)dq2;
  if (ptr_bits & (dtype == TS_F32 ? 3u : 1u)) return TS_ERR_ALIGN;
  // the bf16 path reads rows as 16-byte vectors; rows that are not aligned for that take the other path
  const bool fast = ts::nce_bf16_path(c, tau, dtype) && (ptr_bits & 15u) == 0;
  hipStream_t st = (hipStream_t)stream;
  const int pairs = q2 ? 2 : 1;
  if (n == 0) {
    // cross entropy over zero rows: mean of nothing = NaN, as torch gives
    return ts::launch_sum_scale((const float*)workspace, 0, 1.f, 0.f, loss_out, st);
  }
  ts::NceArgs args;
  for (int p = 0; p < 2; ++p) {
    ts::nce_clear_pieces(args.p[p]);
    const int src = p < pairs ? p : 0;
    args.p[p].q = src ? q2 : q1;
    args.p[p].k = src ? k2 : k1;
    args.p[p].dq = src ? dq2 : dq1;
  }
  if (!fast) return ts::nce_general_launch(args, pairs, n, c, tau, workspace, loss_out, dtype, st);
  return ts::nce_launch(args, pairs, n, c, tau, workspace, loss_out, dtype, st);
}

int ts_infonce_pieces_fwd_bwd(const void* const* q1_pieces, const void* const* k1_pieces, void* const* dq1_pieces,
                              const void* const* q2_pieces, const void* const* k2_pieces, void* const* dq2_pieces,
                              const int64_t* piece_rows, int n_pieces, int64_t c, float tau, void* workspace,
                              float* loss_out, int dtype, ts_stream_t stream) {
  if (!q1_pieces || !k1_pieces || !piece_rows || !workspace || !loss_out) return TS_ERR_ARG;
  if ((q2_pieces == nullptr) != (k2_pieces == nullptr)) return TS_ERR_ARG;
  if (n_pieces < 1 || n_pieces > ts::kNceMaxPieces) return TS_ERR_RANGE;
  if (!(tau > 0.f) || c < 1) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (c > 512) return TS_ERR_RANGE;
  if ((uintptr_t)workspace & 255u) return TS_ERR_ALIGN;
  const int pairs = q2_pieces ? 2 : 1;
  bool fast = ts::nce_bf16_path(c, tau, dtype);
  const uintptr_t elem_mask = dtype == TS_F32 ? 3u : 1u;
  ts::NceArgs args;
  int64_t n = 0;
  for (int p = 0; p < 2; ++p) {
    ts::NcePair& P = args.p[p];
    ts::nce_clear_pieces(P);
    if (p >= pairs) continue;
    const void* const* qs = p ? q2_pieces : q1_pieces;
    const void* const* ks = p ? k2_pieces : k1_pieces;
    void* const* ds = p ? dq2_pieces : dq1_pieces;
    const bool want = ds && ds[0];
    int64_t rows = 0;
    for (int i = 0; i < n_pieces; ++i) {
      if (piece_rows[i] <= 0 || !qs[i] || !ks[i]) return TS_ERR_ARG;
      if (want != (ds && ds[i] != nullptr)) return TS_ERR_ARG;
      const uintptr_t bits = (uintptr_t)qs[i] | (uintptr_t)ks[i] | (uintptr_t)(want ? ds[i] : nullptr);
      if (bits & elem_mask) return TS_ERR_ALIGN;
      if (bits & 15u) fast = false;  // the bf16 path reads rows as 16-byte vectors
      P.row0[i] = rows;
      P.qp[i] = qs[i];
      P.kp[i] = ks[i];
      P.dqp[i] = want ? ds[i] : nullptr;
      rows += piece_rows[i];
    }
    P.n_pieces = n_pieces;
    n = rows;
  }
  if (n > (1 << 24)) return TS_ERR_RANGE;
  if (!fast) return ts::nce_general_launch(args, pairs, n, c, tau, workspace, loss_out, dtype, (hipStream_t)stream);
  return ts::nce_launch(args, pairs, n, c, tau, workspace, loss_out, dtype, (hipStream_t)stream);
}

}  // extern "C"
