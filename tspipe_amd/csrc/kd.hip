// Distillation row losses, forward and backward fused:
//   KD soft target   KL(softmax(t/T) || softmax(s/T)) over rows selected by a mask,
//   hard-label CE    cross entropy of softmax(s) against integer labels with an
//                    ignore index, optionally in the same pass over the rows.
// A "group" of threads owns a row and holds it in registers: 16/32/64 lanes of
// a wavefront for narrow rows, a 256-, 512- or 1024-thread workgroup for rows
// of up to 8192 16-byte vectors (vocabulary-sized rows included); wider rows,
// and long rows whose operands are aligned differently, are cut into parts
// handled by short-lived workgroups in two launches.
// Accumulation is fp32 in the log2 domain (v_exp_f32 / v_log_f32); storage is
// fp32, bf16 or fp16.
#include <mutex>

#include "common.h"

namespace ts {

// Scratch of ts_kd_fwd_bwd_static: one copy per GPU, held until the process
// ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels are handed the address it returns.
constexpr size_t kKdStaticScratchBytes = (size_t)1 << 20;
static __device__ __align__(256) unsigned char kd_static_scratch[kKdStaticScratchBytes];
constexpr int kKdMaxDevices = 64;
static std::mutex g_kd_scratch_lock;
static void* g_kd_scratch_ptr[kKdMaxDevices];  // device address of the array, per device ordinal

// Address of the current device's copy of the scratch array (looked up once
// per device); nullptr with *rc set when the runtime refuses.
static void* kd_static_scratch_ptr(int* rc) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kKdMaxDevices) {
    set_last_hip_error((int)e);
    *rc = e != hipSuccess ? TS_ERR_LAUNCH : TS_ERR_RANGE;
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(g_kd_scratch_lock);
  if (!g_kd_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(kd_static_scratch));
    if (e != hipSuccess || !p) {
      set_last_hip_error((int)e);
      *rc = TS_ERR_LAUNCH;
      return nullptr;
    }
    g_kd_scratch_ptr[dev] = p;
  }
  return g_kd_scratch_ptr[dev];
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -3.0e38f;  // finite stand-in for -inf: keeps 2^((m_old - m_new) k) NaN-free

// Online soft-max state of part of a row.  Maxima are kept in raw logit
// units; k = inv_T * log2(e) scales differences into the log2 domain.
//   teacher: m = max t, z = sum 2^((t-m)k), a = sum 2^((t-m)k) (t - s)
//   student: m = max s, z = sum 2^((s-m)k), z1 = sum 2^((s-m) log2e)   (z1: temperature 1, for the CE term)
struct TStat {
  float m, z, a;
};
struct SStat {
  float m, z, z1;
};

// acc + w * (t - s) for the sum p (t - s) of the KD term.  A teacher logit of
// -inf (a masked vocabulary entry) has weight w = 2^(-inf) = 0 and must
// contribute nothing, as F.kl_div's xlogy gives, where 0 * (-inf) would be
// NaN: the difference is kept finite from below (fmaxf also turns the NaN of
// -inf - -inf into the bound).  +inf (student -inf under a positive teacher
// weight) stays: the reference's loss is +inf there too.
__device__ __forceinline__ float acc_weighted_diff(float w, float t, float s, float acc) {
  return fmaf(w, fmaxf(t - s, -3.4028234e38f), acc);
}

__device__ __forceinline__ TStat tstat_init() { return TStat{kNegBig, 0.f, 0.f}; }
__device__ __forceinline__ SStat sstat_init() { return SStat{kNegBig, 0.f, 0.f}; }

__device__ __forceinline__ TStat merge(TStat p, TStat q, float k) {
  const float m = fmaxf(p.m, q.m);
  const float rp = fast_exp2((p.m - m) * k), rq = fast_exp2((q.m - m) * k);
  return TStat{m, p.z * rp + q.z * rq, p.a * rp + q.a * rq};
}

template <bool CE>
__device__ __forceinline__ SStat merge(SStat p, SStat q, float k) {
  const float m = fmaxf(p.m, q.m);
  const float dp = p.m - m, dq = q.m - m;
  SStat r{m, p.z * fast_exp2(dp * k) + q.z * fast_exp2(dq * k), 0.f};
  if (CE) r.z1 = p.z1 * fast_exp2(dp * kLog2e) + q.z1 * fast_exp2(dq * kLog2e);
  return r;
}

// Reduction over WIDTH (<= 64, power of two) adjacent lanes.
template <int WIDTH, bool CE>
__device__ __forceinline__ void lane_reduce(TStat& t, SStat& s, float k) {
#pragma unroll
  for (int off = WIDTH / 2; off > 0; off >>= 1) {
    const TStat ot{__shfl_xor(t.m, off, kWave), __shfl_xor(t.z, off, kWave), __shfl_xor(t.a, off, kWave)};
    SStat os{__shfl_xor(s.m, off, kWave), __shfl_xor(s.z, off, kWave), 0.f};
    if (CE) os.z1 = __shfl_xor(s.z1, off, kWave);
    t = merge(t, ot, k);
    s = merge<CE>(s, os, k);
  }
}

// Folds N (teacher, student) logit pairs into the states.  The block's own
// maxima are taken first, so each element costs one fma and one exp2 per
// operand (two for the student when the CE term is on), and the running
// states are rescaled once per block.
template <int N, bool CE>
__device__ __forceinline__ void fold(TStat& st, SStat& ss, const float (&t)[N], const float (&s)[N], float k) {
  float mt = t[0], ms = s[0];
#pragma unroll
  for (int i = 1; i < N; ++i) {
    mt = fmaxf(mt, t[i]);
    ms = fmaxf(ms, s[i]);
  }
  // a block of nothing but -inf (masked vocabulary entries) keeps a finite
  // reference point, so that its terms are 2^(-inf) = 0 and not 2^(inf - inf)
  mt = fmaxf(mt, kNegBig);
  ms = fmaxf(ms, kNegBig);
  const float mtk = mt * k, msk = ms * k, ms1 = ms * kLog2e;
  float zt = 0.f, at = 0.f, zs = 0.f, z1 = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float et = fast_exp2(fmaf(t[i], k, -mtk));
    zt += et;
    at = acc_weighted_diff(et, t[i], s[i], at);
    zs += fast_exp2(fmaf(s[i], k, -msk));
    if (CE) z1 += fast_exp2(fmaf(s[i], kLog2e, -ms1));
  }
  st = merge(st, TStat{mt, zt, at}, k);
  ss = merge<CE>(ss, SStat{ms, zs, z1}, k);
}

// Everything a row kernel needs; passed by value.
// The logits may come as up to kKdMaxPieces row blocks (micro-batch outputs
// that were never concatenated): piece p holds rows piece_row0[p] ..
// piece_row0[p+1]-1 of the batch, contiguous with the common leading
// dimensions.  n_pieces == 0 means the single matrices s / t / grad.
constexpr int kKdMaxPieces = 8;

struct KdArgs {
  const void* s;
  const void* t;
  const uint8_t* mask;    // KD row selection, may be null (all rows)
  const int64_t* labels;  // CE labels, may be null (no CE term)
  int64_t ignore_index;
  int64_t n_rows, V, ld_s, ld_t, ld_g;
  float k;          // inv_T * log2(e)
  float kd_gscale;  // kd_scale * inv_T   (gradient factor of the KD term before the 1/B)
  float ce_weight;
  int t_pow;        // the temperature when it is exactly 1, 2 or 4 (then 2^x at temperature 1 is a power of 2^x at T), else 0
  const int* counts;  // device: [0] KD rows, [1] CE rows, [2] rows with any term; null = all n_rows carry KD only
  int self_count;     // counts is null although a mask or labels select rows: whoever needs the numbers of KD / CE rows counts them
  int split_grid;     // long rows under a mask: the grid has a second half of workgroups that zero-fill the rows without a term
  float* row_kd;      // per-row KD loss terms (0 for unselected rows)
  float* row_ce;      // per-row CE loss terms
  void* grad;         // may be null
  int n_pieces;
  int64_t piece_row0[kKdMaxPieces];
  const void* s_piece[kKdMaxPieces];
  const void* t_piece[kKdMaxPieces];
  void* g_piece[kKdMaxPieces];  // all null or all set
};

// Row pointers.  The piece is found with a chain of selects rather than an
// indexed load, because a wavefront may hold several rows.
template <typename T>
struct KdRowPtrs {
  const T* s;
  const T* t;
  T* g;
};

template <typename T>
__device__ __forceinline__ KdRowPtrs<T> kd_row_ptrs(const KdArgs& a, int64_t row) {
  KdRowPtrs<T> r;
  if (a.n_pieces == 0) {
    r.s = reinterpret_cast<const T*>(a.s) + row * a.ld_s;
    r.t = reinterpret_cast<const T*>(a.t) + row * a.ld_t;
    r.g = a.grad ? reinterpret_cast<T*>(a.grad) + row * a.ld_g : nullptr;
    return r;
  }
  const void* sb = a.s_piece[0];
  const void* tb = a.t_piece[0];
  void* gb = a.g_piece[0];
  int64_t r0 = 0;
#pragma unroll
  for (int i = 1; i < kKdMaxPieces; ++i) {
    const bool ge = i < a.n_pieces && row >= a.piece_row0[i];
    sb = ge ? a.s_piece[i] : sb;
    tb = ge ? a.t_piece[i] : tb;
    gb = ge ? a.g_piece[i] : gb;
    r0 = ge ? a.piece_row0[i] : r0;
  }
  const int64_t local = row - r0;
  r.s = reinterpret_cast<const T*>(sb) + local * a.ld_s;
  r.t = reinterpret_cast<const T*>(tb) + local * a.ld_t;
  r.g = gb ? reinterpret_cast<T*>(gb) + local * a.ld_g : nullptr;
  return r;
}

__device__ __forceinline__ bool kd_has_grad(const KdArgs& a) { return a.n_pieces ? a.g_piece[0] != nullptr : a.grad != nullptr; }

struct RowJob {
  bool kd, ce;
  int64_t label;
};

__device__ __forceinline__ RowJob row_job(const KdArgs& a, int64_t row) {
  RowJob j;
  j.kd = a.mask ? (a.mask[row] != 0) : true;
  j.ce = false;
  j.label = 0;
  if (a.labels) {
    j.label = a.labels[row];
    j.ce = (j.label != a.ignore_index) && j.label >= 0 && j.label < a.V;
  }
  return j;
}

// Final per-row numbers from the merged states.
struct RowFinal {
  float lse_t, lse_s, lse1;  // log2 domain
  float g_kd, g_ce;          // gradient factors (0 when the term is off for this row)
};

// Number of rows whose label selects a class (not the ignore index, inside
// [0, V)), counted by the calling workgroup like mask_count_block.
template <int NT>
__device__ __forceinline__ float label_count_block(const int64_t* __restrict__ labels, int64_t n, int64_t ignore_index,
                                                   int64_t V, float* lds) {
  int c = 0;
  constexpr int kInFlight = 4;  // loads per thread and trip
  for (int64_t i0 = threadIdx.x; i0 < n; i0 += (int64_t)NT * kInFlight) {
    int64_t l[kInFlight];
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) {
      const int64_t i = i0 + (int64_t)j * NT;
      l[j] = i < n ? labels[i] : ignore_index;
    }
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) c += (l[j] != ignore_index && l[j] >= 0 && l[j] < V) ? 1 : 0;
  }
  return block_sum<NT / kWave>((float)c, lds);
}

template <typename T, bool CE>
__device__ __forceinline__ RowFinal finish_row(const KdArgs& a, const RowJob& j, int64_t row, const TStat& st,
                                               const SStat& ss, const T* srow, bool writer, float n_kd_counted = 0.f,
                                               float n_ce_counted = 0.f) {
  RowFinal f;
  f.lse_t = st.m * a.k + log2f(st.z);
  f.lse_s = ss.m * a.k + log2f(ss.z);
  f.lse1 = CE ? ss.m * kLog2e + log2f(ss.z1) : 0.f;
  const float n_kd = a.self_count ? n_kd_counted : (a.counts ? (float)a.counts[0] : (float)a.n_rows);
  f.g_kd = j.kd ? a.kd_gscale / n_kd : 0.f;
  f.g_ce = (CE && j.ce) ? a.ce_weight / (a.self_count ? n_ce_counted : (float)a.counts[1]) : 0.f;
  if (writer) {
    a.row_kd[row] = j.kd ? kLn2 * (a.k * st.a / st.z - f.lse_t + f.lse_s) : 0.f;
    if (CE) a.row_ce[row] = j.ce ? kLn2 * (f.lse1 - to_f32(srow[j.label]) * kLog2e) : 0.f;
  }
  return f;
}

template <typename T, bool CE>
__device__ __forceinline__ T grad_one(T tv, T sv, bool hit, float k, const RowFinal& f) {
  const float sf = to_f32(sv);
  const float p = fast_exp2(fmaf(to_f32(tv), k, -f.lse_t));
  const float q = fast_exp2(fmaf(sf, k, -f.lse_s));
  float g = f.g_kd * (q - p);
  if (CE) {
    const float r = fast_exp2(fmaf(sf, kLog2e, -f.lse1));
    g = fmaf(f.g_ce, r - (hit ? 1.f : 0.f), g);
  }
  return from_f32<T>(g);
}

template <typename T, int GROUP>
__device__ __forceinline__ void zero_row(T* grow, int64_t V, int gtid) {
  constexpr int VEC = Vec16<T>::N;
  const uint32_t mis = (uint32_t)((uintptr_t)grow & 15u);
  int64_t head = (int64_t)(((16u - mis) & 15u) / sizeof(T));
  if (head > V) head = V;
  const int64_t nvec = (V - head) / VEC, tail0 = head + nvec * VEC;
  const T zero = from_f32<T>(0.f);
  Vec16<T> z;
#pragma unroll
  for (int i = 0; i < VEC; ++i) z.v[i] = zero;
  for (int64_t i = gtid; i < head; i += GROUP) grow[i] = zero;
  for (int64_t v = gtid; v < nvec; v += GROUP) store16(grow + head + v * VEC, z);
  for (int64_t i = tail0 + gtid; i < V; i += GROUP) grow[i] = zero;
}

struct RowGeom {
  int64_t head, nvec, tail0;
};

// Split of a row into scalar head, 16-byte vectors and scalar tail by the
// common misalignment of its pointers; everything is "head" when they disagree.
template <typename T>
__device__ __forceinline__ RowGeom row_geom(const T* srow, const T* trow, const T* grow, int64_t V) {
  constexpr int VEC = Vec16<T>::N;
  const uint32_t mis_s = (uint32_t)((uintptr_t)srow & 15u), mis_t = (uint32_t)((uintptr_t)trow & 15u);
  const uint32_t mis_g = grow ? (uint32_t)((uintptr_t)grow & 15u) : mis_s;
  RowGeom g;
  g.head = (mis_s == mis_t && mis_s == mis_g) ? (int64_t)(((16u - mis_s) & 15u) / sizeof(T)) : V;
  if (g.head > V) g.head = V;
  g.nvec = (V - g.head) / VEC;
  g.tail0 = g.head + g.nvec * VEC;
  return g;
}

// ---------------------------------------------------------------------------
// Rows of up to 8192 vectors: one launch.  The row pair is held in registers
// between the statistics and the gradient (KREG 16-byte vectors per thread
// and operand, all loads issued up front), so each logit is read once; the
// launcher guarantees ceil(V / VEC) + 1 <= KREG * GROUP.
// ---------------------------------------------------------------------------
template <typename T, int BLOCK, int GROUP, int KREG, bool CE>
__global__ __launch_bounds__(BLOCK, (KREG * GROUP > 1024 ? 4 : 1)) void kd_rows_kernel(
    const KdArgs a, const int* __restrict__ sel_rows) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int NW = GROUP / kWave;  // wavefronts per group (0 for sub-wavefront groups)
  __shared__ TStat lds_t[BLOCK / kWave];
  __shared__ SStat lds_s[BLOCK / kWave];
  __shared__ float lds_cnt[BLOCK / kWave];

  const int gtid = threadIdx.x % GROUP;
  int64_t row = (int64_t)blockIdx.x * (BLOCK / GROUP) + threadIdx.x / GROUP;
  // With GROUP == BLOCK the whole workgroup shares one row, so the early
  // exits below are uniform; smaller groups never reach a __syncthreads and
  // only shuffle among their own lanes.
  // Short rows (several to a workgroup) without a counting launch in front:
  // every workgroup counts the mask and the labels itself, all of its threads
  // together, before any of them leaves (a few hundred rows: one load each).
  float n_kd_counted = 0.f, n_ce_counted = 0.f;
  if (GROUP < BLOCK && a.self_count) {
    n_kd_counted = a.mask ? mask_count_block<BLOCK>(a.mask, a.n_rows, lds_cnt) : (float)a.n_rows;
    if (CE && a.labels) n_ce_counted = label_count_block<BLOCK>(a.labels, a.n_rows, a.ignore_index, a.V, lds_cnt);
  }
  if (sel_rows || a.split_grid) {
    // Masked long rows (one row per workgroup, grid of 2 n_rows): the first
    // n_rows workgroups take the rows that carry a loss term, so that the
    // long-running ones all start first; the next n_rows zero-fill the rows
    // that carry none (one row each: eight rows per workgroup were slower,
    // 74.6 against 72.1 us on 4096 x 30522 under a 15 % mask).  (Interleaving the two kinds, singly or in runs of
    // eight, was measured slower than this order.)  With a compacted row list
    // (built by the counting launch, which a cross-entropy term needs anyway)
    // workgroup i of the first half takes the i-th such row; without one it
    // takes row i if that carries a term and ends at once otherwise.
    if (row >= a.n_rows) {
      row -= a.n_rows;
      const RowJob j0 = row_job(a, row);
      if (j0.kd || j0.ce) return;
    } else if (sel_rows) {
      if (row >= a.counts[2]) return;
      row = sel_rows[row];
    } else {
      const RowJob j0 = row_job(a, row);
      if (!j0.kd && !j0.ce) return;
    }
  }
  if (row >= a.n_rows) return;
  const KdRowPtrs<T> rp = kd_row_ptrs<T>(a, row);
  const T* srow = rp.s;
  const T* trow = rp.t;
  T* grow = rp.g;
  const RowJob job = row_job(a, row);
  const int64_t V = a.V;

  if (!job.kd && !job.ce) {
    if (gtid == 0) {
      a.row_kd[row] = 0.f;
      if (CE) a.row_ce[row] = 0.f;
    }
    if (grow) zero_row<T, GROUP>(grow, V, gtid);
    return;
  }

  const RowGeom g = row_geom<T>(srow, trow, grow, V);
  Vec16<T> rt[KREG], rs[KREG];
#ifdef TS_KD_ROWS_IN_LDS
  // Measurement variant, not part of the default build: the 512-thread
  // long-row instantiation for 16-bit logits parks the row pair in LDS (2 x 64
  // KB, one workgroup per CU) instead of in registers, every lane reading back
  // the vectors it wrote, one pair at a time in each of the three walks.
  constexpr bool kStage = BLOCK == 512 && KREG * GROUP > 1024 && sizeof(T) == 2;
  __shared__ u32x4 stage_t[kStage ? KREG * GROUP : 1], stage_s[kStage ? KREG * GROUP : 1];
#else
  constexpr bool kStage = false;
  u32x4* const stage_t = nullptr;
  u32x4* const stage_s = nullptr;
#endif
#pragma unroll
  for (int j = 0; j < KREG; ++j) {
    const int64_t v = gtid + (int64_t)j * GROUP;
    if (v < g.nvec) {
      if constexpr (kStage) {
        const Vec16<T> lt = load16(trow + g.head + v * VEC), ls = load16(srow + g.head + v * VEC);
        __builtin_memcpy(&stage_t[v], &lt, 16);
        __builtin_memcpy(&stage_s[v], &ls, 16);
      } else {
        // The logits are read once: non-temporal loads.  On working sets beyond the last-level cache,
        // us per call: 32768 x 1000 fp32 75.0 -> 71.0, 16384 x 4000 fp32 144 -> 128, 8192 x 16000 fp32
        // 283 -> 264, 4096 x 30522 bf16 with and without a mask unchanged.  (A loop on one set of logits
        // that fits that cache loses, 8192 x 4096 bf16 45 -> 52: its own plain loads were what kept the
        // set there from call to call.)
        rt[j] = load16_stream(trow + g.head + v * VEC);
        rs[j] = load16_stream(srow + g.head + v * VEC);
      }
    }
  }
  // No counting launch ran in front (long rows under a mask and / or with
  // labels): the numbers of rows with a KD and with a CE term, which scale the
  // gradient, are counted here while the row's loads are in flight.  One row per workgroup in that case, so the
  // branch is uniform.
  if (GROUP == BLOCK && a.self_count) {
    n_kd_counted = a.mask ? mask_count_block<BLOCK>(a.mask, a.n_rows, lds_cnt) : (float)a.n_rows;
    if (CE && a.labels) n_ce_counted = label_count_block<BLOCK>(a.labels, a.n_rows, a.ignore_index, a.V, lds_cnt);
  }

  // Rows whose operands share one alignment (the usual case): all but a few
  // end elements are 16-byte vectors held in registers, and each of those end
  // elements gets a lane of its own.
  // the long-row instantiation is only launched on rows of this kind (checked on the host)
  constexpr bool kAlignedOnly = KREG * GROUP > 1024;
  const int64_t ntail = V - g.tail0;
  if (kAlignedOnly || (g.head < VEC && ntail < VEC)) {
    // The packed row pair stays in registers and is walked three times
    // (maxima, sums, gradient).  (Keeping the exponentials BESIDE the logits
    // doubles the registers and was measured slower: occupancy is what hides
    // the load latency here.)
    const bool has_h = gtid < g.head, has_t = gtid < ntail;
    float eh_t = kNegBig, eh_s = kNegBig, el_t = kNegBig, el_s = kNegBig;  // end elements: head, last
    if (has_h) {
      eh_t = to_f32(trow[gtid]);
      eh_s = to_f32(srow[gtid]);
    }
    if (has_t) {
      el_t = to_f32(trow[g.tail0 + gtid]);
      el_s = to_f32(srow[g.tail0 + gtid]);
    }
    // Each walk starts from registers the compiler can assume nothing about;
    // otherwise it would unpack the row once and keep all the fp32 values.
    auto fresh = [&](int j) {
      if constexpr (kStage) {
        __builtin_memcpy(&rt[j], &stage_t[gtid + j * GROUP], 16);
        __builtin_memcpy(&rs[j], &stage_s[gtid + j * GROUP], 16);
        return;
      }
      u32x4 bt, bs;
      __builtin_memcpy(&bt, &rt[j], 16);
      __builtin_memcpy(&bs, &rs[j], 16);
      asm volatile("" : "+v"(bt), "+v"(bs));
      __builtin_memcpy(&rt[j], &bt, 16);
      __builtin_memcpy(&rs[j], &bs, 16);
    };
    float mt = fmaxf(eh_t, el_t), ms = fmaxf(eh_s, el_s);
#pragma unroll
    for (int j = 0; j < KREG; ++j) {
      if (gtid + j * GROUP < (int)g.nvec) {
        if constexpr (kStage) fresh(j);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          mt = fmaxf(mt, to_f32(rt[j].v[i]));
          ms = fmaxf(ms, to_f32(rs[j].v[i]));
        }
      }
      // one vector pair at a time: unpacking all of them ahead would double the registers
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int off = (GROUP < kWave ? GROUP : kWave) / 2; off > 0; off >>= 1) {
      mt = fmaxf(mt, __shfl_xor(mt, off, kWave));
      ms = fmaxf(ms, __shfl_xor(ms, off, kWave));
    }
    const int w = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (NW > 1) {
      if (lane == 0) {
        lds_t[w].m = mt;
        lds_s[w].m = ms;
      }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < NW; ++i) {
        mt = fmaxf(mt, lds_t[i].m);
        ms = fmaxf(ms, lds_s[i].m);
      }
    }
    const float mtk = mt * a.k, msk = ms * a.k, ms1 = ms * kLog2e;
    // The CE term wants 2^((s - m) log2e), the KD term has 2^((s - m) log2e / T):
    // for T = 1, 2, 4 the first is a power of the second, two multiplies at
    // most instead of a v_exp_f32 (a quarter-rate instruction in a kernel
    // that is bound by its vector arithmetic).  t_pow is uniform.
    const int t_pow = CE ? a.t_pow : 0;
    auto e1_of = [&](float sv, float es) {
      if (t_pow == 0) return fast_exp2(fmaf(sv, kLog2e, -ms1));
      float e = es;
      if (t_pow >= 2) e *= e;
      if (t_pow == 4) e *= e;
      return e;
    };
    // fp32 rows: the second walk leaves its exponentials where the logits
    // were (the student's logit stays when the CE term needs it at temperature
    // 1), so the gradient walk takes none again.  16-bit rows retake them: a
    // 16-bit slot would round them, and p_s - p_t cancels.
    constexpr bool kKeep = sizeof(T) == 4;
    float zt = 0.f, at = 0.f, zs = 0.f, z1 = 0.f;
    // a missing end element contributes 2^(-huge) = 0; most wavefronts have none at all
    if (__any(has_h || has_t)) {
      auto add = [&](float tv, float sv) {
        const float et = fast_exp2(fmaf(tv, a.k, -mtk));
        const float es = fast_exp2(fmaf(sv, a.k, -msk));
        zt += et;
        zs += es;
        at = acc_weighted_diff(et, tv, sv, at);
        if (CE) z1 += e1_of(sv, es);
      };
      add(eh_t, eh_s);
      add(el_t, el_s);
    }
#pragma unroll
    for (int j = 0; j < KREG; ++j) {
      if (gtid + j * GROUP < (int)g.nvec) {
        fresh(j);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const float tv = to_f32(rt[j].v[i]), sv = to_f32(rs[j].v[i]);
          const float et = fast_exp2(fmaf(tv, a.k, -mtk));
          const float es = fast_exp2(fmaf(sv, a.k, -msk));
          zt += et;
          zs += es;
          at = acc_weighted_diff(et, tv, sv, at);
          if (CE) z1 += e1_of(sv, es);
          if constexpr (kKeep) {
            rt[j].v[i] = et;
            if (!CE) rs[j].v[i] = es;
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int off = (GROUP < kWave ? GROUP : kWave) / 2; off > 0; off >>= 1) {
      zt += __shfl_xor(zt, off, kWave);
      zs += __shfl_xor(zs, off, kWave);
      at += __shfl_xor(at, off, kWave);
      if (CE) z1 += __shfl_xor(z1, off, kWave);
    }
    if (NW > 1) {
      // .m of both arrays is still being read by slower wavefronts; the sums go into the other fields
      if (lane == 0) {
        lds_t[w].z = zt;
        lds_t[w].a = at;
        lds_s[w].z = zs;
        lds_s[w].z1 = z1;
      }
      __syncthreads();
      zt = at = zs = z1 = 0.f;
#pragma unroll
      for (int i = 0; i < NW; ++i) {
        zt += lds_t[i].z;
        at += lds_t[i].a;
        zs += lds_s[i].z;
        z1 += lds_s[i].z1;
      }
    }
    const RowFinal f =
        finish_row<T, CE>(a, job, row, TStat{mt, zt, at}, SStat{ms, zs, z1}, srow, gtid == 0, n_kd_counted, n_ce_counted);
    if (!grow) return;
    // probabilities first and the weight last, as everywhere in this file
    const float rt_ = 1.f / zt, rs_ = 1.f / zs, r1_ = CE ? 1.f / z1 : 0.f;
    const int label = CE ? (int)job.label : -1;  // a row with the CE term has 0 <= label < V
    auto grad_of = [&](float tv, float sv, int col) {
      const float et = fast_exp2(fmaf(tv, a.k, -mtk));
      const float es = fast_exp2(fmaf(sv, a.k, -msk));
      float gv = f.g_kd * fmaf(es, rs_, -(et * rt_));
      if (CE) gv = fmaf(f.g_ce, fmaf(e1_of(sv, es), r1_, col == label ? -1.f : 0.f), gv);
      return from_f32<T>(gv);
    };
    if (has_h) grow[gtid] = grad_of(eh_t, eh_s, gtid);
    if (has_t) grow[g.tail0 + gtid] = grad_of(el_t, el_s, (int)g.tail0 + gtid);
#pragma unroll
    for (int j = 0; j < KREG; ++j) {
      if (gtid + j * GROUP < (int)g.nvec) {
        fresh(j);
        Vec16<T> o;
        const int e0 = (int)g.head + (gtid + j * GROUP) * VEC;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          if constexpr (kKeep) {
            const float pt = rt[j].v[i] * rt_;
            if (CE) {
              const float sv = rs[j].v[i];
              const float es = fast_exp2(fmaf(sv, a.k, -msk));
              const float gv = f.g_kd * fmaf(es, rs_, -pt);
              o.v[i] = fmaf(f.g_ce, fmaf(e1_of(sv, es), r1_, e0 + i == label ? -1.f : 0.f), gv);
            } else {
              o.v[i] = f.g_kd * fmaf(rs[j].v[i], rs_, -pt);
            }
          } else {
            o.v[i] = grad_of(to_f32(rt[j].v[i]), to_f32(rs[j].v[i]), e0 + i);
          }
        }
        store16_stream(grow + e0, o);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    return;
  }

  if constexpr (!kAlignedOnly) {
  TStat st = tstat_init();
  SStat ss = sstat_init();
  {
    float xt1[1], xs1[1];
    for (int64_t i = gtid; i < g.head; i += GROUP) {
      xt1[0] = to_f32(trow[i]);
      xs1[0] = to_f32(srow[i]);
      fold<1, CE>(st, ss, xt1, xs1, a.k);
    }
    for (int64_t i = g.tail0 + gtid; i < V; i += GROUP) {
      xt1[0] = to_f32(trow[i]);
      xs1[0] = to_f32(srow[i]);
      fold<1, CE>(st, ss, xt1, xs1, a.k);
    }
    float xt[VEC], xs[VEC];
#pragma unroll
    for (int j = 0; j < KREG; ++j) {
      if (gtid + (int64_t)j * GROUP < g.nvec) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          xt[i] = to_f32(rt[j].v[i]);
          xs[i] = to_f32(rs[j].v[i]);
        }
        fold<VEC, CE>(st, ss, xt, xs, a.k);
      }
    }
  }

  lane_reduce<(GROUP < kWave ? GROUP : kWave), CE>(st, ss, a.k);
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
      st = merge(st, lds_t[i], a.k);
      ss = merge<CE>(ss, lds_s[i], a.k);
    }
  }

  const RowFinal f = finish_row<T, CE>(a, job, row, st, ss, srow, gtid == 0, n_kd_counted, n_ce_counted);
  if (!grow) return;

  for (int64_t i = gtid; i < g.head; i += GROUP) grow[i] = grad_one<T, CE>(trow[i], srow[i], i == job.label, a.k, f);
  for (int64_t i = g.tail0 + gtid; i < V; i += GROUP)
    grow[i] = grad_one<T, CE>(trow[i], srow[i], i == job.label, a.k, f);
#pragma unroll
  for (int j = 0; j < KREG; ++j) {
    const int64_t v = gtid + (int64_t)j * GROUP;
    if (v < g.nvec) {
      Vec16<T> o;
      const int64_t e0 = g.head + v * VEC;
#pragma unroll
      for (int i = 0; i < VEC; ++i) o.v[i] = grad_one<T, CE>(rt[j].v[i], rs[j].v[i], e0 + i == job.label, a.k, f);
      store16_stream(grow + e0, o);
    }
  }
  }
}

// ---------------------------------------------------------------------------
// Wide rows: a row is cut into parts of kPartVecs 16-byte vectors, one
// short-lived 256-thread workgroup per (row, part), two launches:
//   pass 1, grid = every (row, part): rows with a loss term -> partial state
//           of the part (part_stats[row][part]); other rows -> zero-fill of
//           the part's gradient.  The first kind is bound by exp2 throughput,
//           the second by HBM writes, and they overlap.
//   pass 2, bounded grid walking the (row with a term, part) items of the
//           compacted row list: merges the row's partial states, writes the
//           part's gradient.  Its reads come out of the 256 MB last-level
//           cache when those rows fit there.
// ---------------------------------------------------------------------------
constexpr int kPartBlock = 256;
constexpr int kPartPerThread = 4;
constexpr int kPartVecs = kPartBlock * kPartPerThread;
constexpr int kPass2MaxGrid = 8192;
constexpr int64_t kKdSelfCountRows = 2048;  // short rows: up to this many, every workgroup counts mask and labels itself

struct PartStat {  // 32 bytes
  float mt, zt, at, ms, zs, z1, pad0, pad1;
};

template <int NT>
__device__ __forceinline__ void kd_count_block(const KdArgs& a, int* __restrict__ counts, int* __restrict__ sel_rows);

// A row without a loss term: zero loss entries, and this part of its gradient row zero-filled.
template <typename T, bool CE>
__device__ __forceinline__ void kd_zero_part(const KdArgs& a, int64_t row, int part, int parts) {
  constexpr int VEC = Vec16<T>::N;
  const int tid = threadIdx.x;
  const int64_t V = a.V;
  const int64_t v0 = (int64_t)part * kPartVecs;
  if (part == 0 && tid == 0) {
    a.row_kd[row] = 0.f;
    if (CE) a.row_ce[row] = 0.f;
  }
  if (!kd_has_grad(a)) return;
  T* grow = kd_row_ptrs<T>(a, row).g;
  const uint32_t mis = (uint32_t)((uintptr_t)grow & 15u);
  int64_t head = (int64_t)(((16u - mis) & 15u) / sizeof(T));
  if (head > V) head = V;
  const int64_t nvec = (V - head) / VEC, tail0 = head + nvec * VEC;
  const T zero = from_f32<T>(0.f);
  Vec16<T> z;
#pragma unroll
  for (int i = 0; i < VEC; ++i) z.v[i] = zero;
  if (part == 0)
    for (int64_t i = tid; i < head; i += kPartBlock) grow[i] = zero;
  if (part == parts - 1)
    for (int64_t i = tail0 + tid; i < V; i += kPartBlock) grow[i] = zero;
#pragma unroll
  for (int j = 0; j < kPartPerThread; ++j) {
    const int64_t v = v0 + tid + j * kPartBlock;
    if (v < nvec) store16(grow + head + v * VEC, z);
  }
}

// With count_out set, workgroup 0 does the row counting and compaction that
// pass 2 and the final reduction need (nothing in pass 1 reads them), and the
// (row, part) items start at workgroup 1.
template <typename T, bool CE>
__global__ __launch_bounds__(kPartBlock) void kd_wide_pass1_kernel(const KdArgs a, int parts,
                                                                   PartStat* __restrict__ part_stats,
                                                                   int* __restrict__ count_out,
                                                                   int* __restrict__ sel_rows_out) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ TStat lds_t[kPartBlock / kWave];
  __shared__ SStat lds_s[kPartBlock / kWave];
  if (count_out && blockIdx.x == 0) {
    kd_count_block<kPartBlock>(a, count_out, sel_rows_out);
    return;
  }
  const int64_t item = (int64_t)blockIdx.x - (count_out ? 1 : 0);
  const int64_t row = item / parts;
  const int part = (int)(item % parts);
  const int tid = threadIdx.x;
  const int64_t v0 = (int64_t)part * kPartVecs;
  const int64_t V = a.V;
  const RowJob job = row_job(a, row);

  if (!job.kd && !job.ce) {
    kd_zero_part<T, CE>(a, row, part, parts);
    return;
  }

  const KdRowPtrs<T> rp = kd_row_ptrs<T>(a, row);
  const T* srow = rp.s;
  const T* trow = rp.t;
  // the row is cut by the alignment of s and t alone; pass 2 cuts it the same way
  const RowGeom g = row_geom<T>(srow, trow, nullptr, V);
  Vec16<T> rt[kPartPerThread], rs[kPartPerThread];
#pragma unroll
  for (int j = 0; j < kPartPerThread; ++j) {
    const int64_t v = v0 + tid + j * kPartBlock;
    if (v < g.nvec) {
      rt[j] = load16(trow + g.head + v * VEC);
      rs[j] = load16(srow + g.head + v * VEC);
    }
  }
  // Ragged ends of the row (fewer than VEC elements each, unless the rows are
  // misaligned against each other and everything is "head"): folded into
  // per-thread states the slow way.
  TStat st = tstat_init();
  SStat ss = sstat_init();
  float xt1[1], xs1[1];
  if (part == 0) {
    for (int64_t i = tid; i < g.head; i += kPartBlock) {
      xt1[0] = to_f32(trow[i]);
      xs1[0] = to_f32(srow[i]);
      fold<1, CE>(st, ss, xt1, xs1, a.k);
    }
  }
  if (part == parts - 1) {
    for (int64_t i = g.tail0 + tid; i < V; i += kPartBlock) {
      xt1[0] = to_f32(trow[i]);
      xs1[0] = to_f32(srow[i]);
      fold<1, CE>(st, ss, xt1, xs1, a.k);
    }
  }
  // Vector body.  The maxima are settled first, over the thread's vectors and
  // then across the wavefront, so that every lane exponentiates against the
  // same reference and the sums combine by plain addition: no per-step
  // rescaling and no exp2 in the cross-lane reduction.
  float mt = st.m, ms = ss.m;
  float ft[kPartPerThread][VEC], fs[kPartPerThread][VEC];
#pragma unroll
  for (int j = 0; j < kPartPerThread; ++j) {
    if (v0 + tid + j * kPartBlock < g.nvec) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        ft[j][i] = to_f32(rt[j].v[i]);
        fs[j][i] = to_f32(rs[j].v[i]);
        mt = fmaxf(mt, ft[j][i]);
        ms = fmaxf(ms, fs[j][i]);
      }
    }
  }
  const float wmt = wave_max(mt), wms = wave_max(ms);
  const float wmtk = wmt * a.k, wmsk = wms * a.k, wms1 = wms * kLog2e;
  // ragged-end sums re-based onto the wavefront's maxima
  const float rbt = fast_exp2((st.m - wmt) * a.k), rbs = fast_exp2((ss.m - wms) * a.k);
  float zt = st.z * rbt, at = st.a * rbt, zs = ss.z * rbs;
  float z1 = CE ? ss.z1 * fast_exp2((ss.m - wms) * kLog2e) : 0.f;
#pragma unroll
  for (int j = 0; j < kPartPerThread; ++j) {
    if (v0 + tid + j * kPartBlock < g.nvec) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float et = fast_exp2(fmaf(ft[j][i], a.k, -wmtk));
        zt += et;
        at = acc_weighted_diff(et, ft[j][i], fs[j][i], at);
        zs += fast_exp2(fmaf(fs[j][i], a.k, -wmsk));
        if (CE) z1 += fast_exp2(fmaf(fs[j][i], kLog2e, -wms1));
      }
    }
  }
  zt = wave_sum(zt);
  at = wave_sum(at);
  zs = wave_sum(zs);
  if (CE) z1 = wave_sum(z1);
  const int w = tid / kWave, lane = tid % kWave;
  if (lane == 0) {
    lds_t[w] = TStat{wmt, zt, at};
    lds_s[w] = SStat{wms, zs, z1};
  }
  __syncthreads();
  if (tid == 0) {
    TStat bt = lds_t[0];
    SStat bs = lds_s[0];
#pragma unroll
    for (int i = 1; i < kPartBlock / kWave; ++i) {
      bt = merge(bt, lds_t[i], a.k);
      bs = merge<CE>(bs, lds_s[i], a.k);
    }
    part_stats[row * parts + part] = PartStat{bt.m, bt.z, bt.a, bs.m, bs.z, bs.z1, 0.f, 0.f};
  }
}

template <typename T, bool CE>
__global__ __launch_bounds__(kPartBlock) void kd_wide_pass2_kernel(const KdArgs a, int parts,
                                                                   const PartStat* __restrict__ part_stats,
                                                                   const int* __restrict__ sel_rows) {
  constexpr int VEC = Vec16<T>::N;
  const int64_t items = (a.counts ? (int64_t)a.counts[2] : a.n_rows) * parts;
  const int tid = threadIdx.x;
  const int64_t V = a.V;

  for (int64_t item = blockIdx.x; item < items; item += gridDim.x) {
    const int64_t row = sel_rows ? (int64_t)sel_rows[item / parts] : item / parts;
    const int part = (int)(item % parts);
    const int64_t v0 = (int64_t)part * kPartVecs;
    const KdRowPtrs<T> rp = kd_row_ptrs<T>(a, row);
    const T* srow = rp.s;
    const T* trow = rp.t;
    T* grow = rp.g;
    const RowJob job = row_job(a, row);
    const RowGeom g = row_geom<T>(srow, trow, nullptr, V);
    const bool gvec = grow && (((uintptr_t)grow & 15u) == ((uintptr_t)srow & 15u));

    Vec16<T> rt[kPartPerThread], rs[kPartPerThread];
    if (grow) {
#pragma unroll
      for (int j = 0; j < kPartPerThread; ++j) {
        const int64_t v = v0 + tid + j * kPartBlock;
        if (v < g.nvec) {
          // second and last read of the row (2048 x 131072 bf16: 511 against 540 us)
          rt[j] = load16_stream(trow + g.head + v * VEC);
          rs[j] = load16_stream(srow + g.head + v * VEC);
        }
      }
    }
    // every thread merges the row's few partial states itself (uniform loads)
    TStat st = tstat_init();
    SStat ss = sstat_init();
    for (int p = 0; p < parts; ++p) {
      const PartStat ps = part_stats[row * parts + p];
      st = merge(st, TStat{ps.mt, ps.zt, ps.at}, a.k);
      ss = merge<CE>(ss, SStat{ps.ms, ps.zs, ps.z1}, a.k);
    }
    const RowFinal f = finish_row<T, CE>(a, job, row, st, ss, srow, part == 0 && tid == 0);
    if (!grow) continue;
    if (part == 0)
      for (int64_t i = tid; i < g.head; i += kPartBlock)
        grow[i] = grad_one<T, CE>(trow[i], srow[i], i == job.label, a.k, f);
    if (part == parts - 1)
      for (int64_t i = g.tail0 + tid; i < V; i += kPartBlock)
        grow[i] = grad_one<T, CE>(trow[i], srow[i], i == job.label, a.k, f);
#pragma unroll
    for (int j = 0; j < kPartPerThread; ++j) {
      const int64_t v = v0 + tid + j * kPartBlock;
      if (v < g.nvec) {
        Vec16<T> o;
        const int64_t e0 = g.head + v * VEC;
#pragma unroll
        for (int i = 0; i < VEC; ++i) o.v[i] = grad_one<T, CE>(rt[j].v[i], rs[j].v[i], e0 + i == job.label, a.k, f);
        if (gvec) {
          store16_stream(grow + e0, o);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) grow[e0 + i] = o.v[i];
        }
      }
    }
  }
}

// Parts a row of V elements of T is cut into (0: the row is narrow enough for
// the single-launch kernel).
template <typename T>
inline int64_t kd_parts(int64_t V) {
  const int64_t vecs = (V + Vec16<T>::N - 1) / Vec16<T>::N + 1;
  if (vecs <= 256 * 4) return 0;
  return (vecs + kPartVecs - 1) / kPartVecs;
}

// counts[0] = rows with the KD term, counts[1] = rows with the CE term,
// counts[2] = rows with either; sel_rows (optional) = indices of the latter in
// ascending order.  One workgroup; thread i owns the i-th contiguous slice.
template <int NT>
__device__ __forceinline__ void kd_count_block(const KdArgs& a, int* __restrict__ counts,
                                               int* __restrict__ sel_rows) {
  __shared__ int scan[NT];
  __shared__ int tot_kd[NT / kWave], tot_ce[NT / kWave];
  const int tid = threadIdx.x;
  const int64_t n = a.n_rows;
  const int64_t per = (n + NT - 1) / NT;
  const int64_t lo = tid * per, hi = (lo + per < n) ? lo + per : n;
  int c_any = 0, c_kd = 0, c_ce = 0;
  if (sel_rows) {
    // a contiguous slice per thread: the row list below comes out in ascending order
    for (int64_t i = lo; i < hi; ++i) {
      const RowJob j = row_job(a, i);
      c_kd += j.kd;
      c_ce += j.ce;
      c_any += (j.kd || j.ce);
    }
  } else {
    // counts only: eight consecutive rows per thread and step (one 8-byte load of the mask, eight labels),
    // four such steps in flight (a contiguous slice per thread, row by row, walks 65536 rows in 31 us)
    const bool wide_mask = !a.mask || ((uintptr_t)a.mask & 7u) == 0;
    const int64_t n8 = wide_mask ? n / 8 : 0;
    const uint64_t* m8 = reinterpret_cast<const uint64_t*>(a.mask);
    constexpr int kInFlight = 4;
    for (int64_t c0 = tid; c0 < n8; c0 += (int64_t)NT * kInFlight) {
      uint64_t mw[kInFlight];
      int64_t lab[kInFlight][8];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const int64_t c = c0 + (int64_t)u * NT;
        mw[u] = 0;
        if (c < n8) {
          mw[u] = a.mask ? m8[c] : ~0ull;
          if (a.labels) {
#pragma unroll
            for (int e = 0; e < 8; ++e) lab[u][e] = a.labels[c * 8 + e];
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const int64_t c = c0 + (int64_t)u * NT;
        if (c < n8) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const bool kd = ((mw[u] >> (8 * e)) & 0xffull) != 0;
            const bool ce = a.labels && lab[u][e] != a.ignore_index && lab[u][e] >= 0 && lab[u][e] < a.V;
            c_kd += kd;
            c_ce += ce;
            c_any += (kd || ce);
          }
        }
      }
    }
    for (int64_t i = n8 * 8 + tid; i < n; i += NT) {
      const RowJob j = row_job(a, i);
      c_kd += j.kd;
      c_ce += j.ce;
      c_any += (j.kd || j.ce);
    }
  }
  // the two plain totals: wavefront sums (exact in float up to 2^24 rows), then one thread adds them
  const float wkd = wave_sum((float)c_kd), wce = wave_sum((float)c_ce);
  if (tid % kWave == 0) {
    tot_kd[tid / kWave] = (int)wkd;
    tot_ce[tid / kWave] = (int)wce;
  }
  if (!sel_rows) {  // uniform: no row list wanted, so no scan either; the third total like the other two
    const float wany = wave_sum((float)c_any);
    if (tid % kWave == 0) scan[tid / kWave] = (int)wany;
    __syncthreads();
    if (tid == 0) {
      int k = 0, c = 0, any = 0;
      for (int i = 0; i < NT / kWave; ++i) {
        k += tot_kd[i];
        c += tot_ce[i];
        any += scan[i];
      }
      counts[0] = k;
      counts[1] = c;
      counts[2] = any;
    }
    return;
  }
  scan[tid] = c_any;
  __syncthreads();
  // inclusive Hillis-Steele scan over the per-thread counts
  for (int off = 1; off < NT; off <<= 1) {
    const int add = (tid >= off) ? scan[tid - off] : 0;
    __syncthreads();
    scan[tid] += add;
    __syncthreads();
  }
  if (tid == 0) {
    int k = 0, c = 0;
    for (int i = 0; i < NT / kWave; ++i) {
      k += tot_kd[i];
      c += tot_ce[i];
    }
    counts[0] = k;
    counts[1] = c;
    counts[2] = scan[NT - 1];
  }
  if (sel_rows) {
    int pos = scan[tid] - c_any;
    for (int64_t i = lo; i < hi; ++i) {
      const RowJob j = row_job(a, i);
      if (j.kd || j.ce) sel_rows[pos++] = (int)i;
    }
  }
}

__global__ __launch_bounds__(1024) void kd_count_kernel(const KdArgs a, int* __restrict__ counts,
                                                        int* __restrict__ sel_rows) {
  kd_count_block<1024>(a, counts, sel_rows);
}

// loss = kd_scale * sum(row_kd) / counts[0] + ce_weight * sum(row_ce) / counts[1], fixed summation order.
// Without counts the workgroup takes the two numbers from the mask (null: all
// n rows carry the KD term) and the labels themselves.
__global__ __launch_bounds__(1024) void kd_finalize_kernel(const float* __restrict__ row_kd,
                                                           const float* __restrict__ row_ce, int64_t n,
                                                           float kd_scale, float ce_weight,
                                                           const int* __restrict__ counts,
                                                           const uint8_t* __restrict__ mask,
                                                           const int64_t* __restrict__ labels, int64_t ignore_index,
                                                           int64_t V, float* __restrict__ out) {
  __shared__ float lds[1024 / kWave];
  const float n_masked = (!counts && mask) ? mask_count_block<1024>(mask, n, lds) : 0.f;
  const float n_labelled = (!counts && row_ce && labels) ? label_count_block<1024>(labels, n, ignore_index, V, lds) : 0.f;
  // 16-byte loads, eight of them in flight per thread and array: one block
  // has to get through the whole array, so the loop is bound by memory latency
  // (65536 rows are two round trips this way)
  const int64_t n4 = n / 4;
  const f32x4* kd4 = reinterpret_cast<const f32x4*>(row_kd);
  const f32x4* ce4 = reinterpret_cast<const f32x4*>(row_ce);
  f32x4 vkd = {0.f, 0.f, 0.f, 0.f}, vce = {0.f, 0.f, 0.f, 0.f};
  constexpr int kInFlight = 8;
  for (int64_t i0 = threadIdx.x; i0 < n4; i0 += 1024 * kInFlight) {
    f32x4 a[kInFlight], c[kInFlight];
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) {
      const int64_t i = i0 + (int64_t)j * 1024;
      a[j] = c[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (i < n4) {
        a[j] = kd4[i];
        if (row_ce) c[j] = ce4[i];
      }
    }
#pragma unroll
    for (int j = 0; j < kInFlight; ++j) {
      vkd += a[j];
      vce += c[j];
    }
  }
  float akd = (vkd[0] + vkd[1]) + (vkd[2] + vkd[3]), ace = (vce[0] + vce[1]) + (vce[2] + vce[3]);
  for (int64_t i = n4 * 4 + threadIdx.x; i < n; i += 1024) {
    akd += row_kd[i];
    if (row_ce) ace += row_ce[i];
  }
  const float skd = block_sum<1024 / kWave>(akd, lds);
  const float sce = block_sum<1024 / kWave>(ace, lds);
  if (threadIdx.x == 0) {
    // 0/0 = NaN for an empty selection, as the reference gives
    float loss = kd_scale * (skd / (counts ? (float)counts[0] : (mask ? n_masked : (float)n)));
    if (row_ce) loss += ce_weight * (sce / (counts ? (float)counts[1] : n_labelled));
    *out = loss;
  }
}

// 1, 2 or 4 when the temperature is exactly that, else 0 (KdArgs::t_pow).
inline int kd_t_pow(float inv_T) { return inv_T == 1.f ? 1 : (inv_T == 0.5f ? 2 : (inv_T == 0.25f ? 4 : 0)); }

struct KdWorkspace {
  int* counts;
  float* row_kd;
  float* row_ce;
  int* sel_rows;
  PartStat* part_stats;
};

inline size_t kd_rows4(int64_t n_rows) { return (size_t)((n_rows * 4 + 31) / 32) * 32; }

inline KdWorkspace kd_carve(void* ws, int64_t n_rows) {
  char* b = reinterpret_cast<char*>(ws);
  const size_t r4 = kd_rows4(n_rows);
  KdWorkspace w;
  w.counts = reinterpret_cast<int*>(b);
  w.row_kd = reinterpret_cast<float*>(b + 32);
  w.row_ce = reinterpret_cast<float*>(b + 32 + r4);
  w.sel_rows = reinterpret_cast<int*>(b + 32 + 2 * r4);
  w.part_stats = reinterpret_cast<PartStat*>(b + 32 + 3 * r4);
  return w;
}

// True when in every row s, t and the gradient sit at the same offset from a
// 16-byte boundary, so that one split into end elements and vectors fits all three.
template <typename T>
inline bool kd_rows_aligned_alike(const KdArgs& a) {
  auto alike = [](const void* x, const void* y) { return (((uintptr_t)x ^ (uintptr_t)y) & 15u) == 0; };
  const int64_t sz = (int64_t)sizeof(T);
  if (((a.ld_s - a.ld_t) * sz) & 15) return false;
  const bool has_g = a.n_pieces ? a.g_piece[0] != nullptr : a.grad != nullptr;
  if (has_g && (((a.ld_s - a.ld_g) * sz) & 15)) return false;
  if (a.n_pieces == 0) return alike(a.s, a.t) && (!has_g || alike(a.s, a.grad));
  for (int p = 0; p < a.n_pieces; ++p)
    if (!alike(a.s_piece[p], a.t_piece[p]) || (has_g && !alike(a.s_piece[p], a.g_piece[p]))) return false;
  return true;
}

template <typename T, bool CE>
int launch_kd_t(KdArgs a, float kd_scale, void* ws, float* loss_out, hipStream_t stream) {
  const KdWorkspace w = kd_carve(ws, a.n_rows);
  const int64_t parts = kd_parts<T>(a.V);
  const bool counted = a.mask || a.labels;  // otherwise all rows carry the KD term and nothing else
  a.counts = counted ? w.counts : nullptr;
  a.row_kd = w.row_kd;
  a.row_ce = w.row_ce;
  const bool compact = parts && counted;
  int rc = TS_OK;
  const int64_t vecs_ = (a.V + Vec16<T>::N - 1) / Vec16<T>::N + 1;
  // Long rows, operands aligned alike: the row pair held in the registers of a
  // 512- or 1024-thread workgroup, one launch.  Under a mask its grid has a
  // second half of workgroups that zero-fill the rows without a term.  The two
  // passes remain for wider or differently aligned rows.
  const bool one_launch = a.n_rows > 0 && parts > 0 && vecs_ <= 1024 * 8 && kd_rows_aligned_alike<T>(a);
  const bool wide = a.n_rows > 0 && parts > 0 && !one_launch;
  // Such rows need no counting launch in front: the numbers the row kernel
  // wants, the counts of rows with a KD and with a CE term, each of its
  // workgroups takes from the mask and the labels themselves (a few
  // kilobytes each), and so does the final reduction.
  // Short rows in small batches (the soft-target benchmark's 256 x 100 with its hard labels) do the
  // same, since there the counting launch is a quarter of the call: 11.4 -> 9.1 us.
  const bool self_count = counted && (one_launch || (parts == 0 && a.n_rows <= kKdSelfCountRows));
  const bool compacted = false;  // (the row kernel can also walk a compacted list of rows with a term)
  a.self_count = self_count ? 1 : 0;
  a.split_grid = (one_launch && self_count && a.mask) ? 1 : 0;
  if (self_count) a.counts = nullptr;
  if (counted && !wide && !self_count) {
    hipLaunchKernelGGL(kd_count_kernel, dim3(1), dim3(1024), 0, stream, a, w.counts,
                       (compact || compacted) ? w.sel_rows : (int*)nullptr);
    rc = check_launch();
    if (rc) return rc;
  }
  if (a.n_rows == 0) {
    hipLaunchKernelGGL(kd_finalize_kernel, dim3(1), dim3(1024), 0, stream, w.row_kd,
                       CE ? w.row_ce : (const float*)nullptr, (int64_t)0, kd_scale, a.ce_weight, a.counts,
                       (const uint8_t*)nullptr, (const int64_t*)nullptr, a.ignore_index, a.V, loss_out);
    return check_launch();
  }
  // 16-byte vectors a row can span, counting a ragged first and last one
  const int64_t vecs = (a.V + Vec16<T>::N - 1) / Vec16<T>::N + 1;
#define TS_KD_LAUNCH(BLOCK, GROUP, KREG)                                                                     \
  hipLaunchKernelGGL((kd_rows_kernel<T, BLOCK, GROUP, KREG, CE>),                                            \
                     dim3((unsigned)((a.n_rows + (BLOCK / GROUP) - 1) / (BLOCK / GROUP))), dim3(BLOCK), 0,   \
                     stream, a, (const int*)nullptr)
  if (vecs <= 16 * 2) {
    TS_KD_LAUNCH(256, 16, 2);
  } else if (vecs <= 32 * 2) {
    TS_KD_LAUNCH(256, 32, 2);
  } else if (vecs <= 64 * 4) {
    TS_KD_LAUNCH(256, 64, 4);
  } else if (parts == 0) {
    TS_KD_LAUNCH(256, 256, 4);
  } else if (one_launch) {
    if (2 * a.n_rows > 0x7fffffffLL) return TS_ERR_RANGE;
    // a second half of zero-filling workgroups only where rows without a term can exist
    const dim3 grid((unsigned)((compacted || a.split_grid) ? 2 * a.n_rows : a.n_rows));
    const int* sel = compacted ? w.sel_rows : nullptr;
    if (vecs <= 512 * 8)
      hipLaunchKernelGGL((kd_rows_kernel<T, 512, 512, 8, CE>), grid, dim3(512), 0, stream, a, sel);
    else
      hipLaunchKernelGGL((kd_rows_kernel<T, 1024, 1024, 8, CE>), grid, dim3(1024), 0, stream, a, sel);
  } else {
    const int64_t items = a.n_rows * parts;
    if (items > 0x7fffffffLL) return TS_ERR_RANGE;
    hipLaunchKernelGGL((kd_wide_pass1_kernel<T, CE>), dim3((unsigned)(items + (counted ? 1 : 0))), dim3(kPartBlock),
                       0, stream, a, (int)parts, w.part_stats, counted ? w.counts : (int*)nullptr,
                       (counted && compact) ? w.sel_rows : (int*)nullptr);
    rc = check_launch();
    if (rc) return rc;
    const int64_t grid2 = items < kPass2MaxGrid ? items : kPass2MaxGrid;
    hipLaunchKernelGGL((kd_wide_pass2_kernel<T, CE>), dim3((unsigned)grid2), dim3(kPartBlock), 0, stream, a,
                       (int)parts, w.part_stats, compact ? w.sel_rows : (const int*)nullptr);
  }
#undef TS_KD_LAUNCH
  rc = check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(kd_finalize_kernel, dim3(1), dim3(1024), 0, stream, w.row_kd, CE ? w.row_ce : (const float*)nullptr,
                     a.n_rows, kd_scale, a.ce_weight, a.counts, self_count ? a.mask : (const uint8_t*)nullptr,
                     self_count ? a.labels : (const int64_t*)nullptr, a.ignore_index, a.V, loss_out);
  return check_launch();
}

template <typename T>
int launch_kd(const KdArgs& a, float kd_scale, void* ws, float* loss_out, hipStream_t stream) {
  return a.labels ? launch_kd_t<T, true>(a, kd_scale, ws, loss_out, stream)
                  : launch_kd_t<T, false>(a, kd_scale, ws, loss_out, stream);
}

}  // namespace ts

extern "C" {

size_t ts_kd_workspace_bytes(int64_t n_rows, int64_t V, int dtype) {
  if (n_rows < 0) n_rows = 0;
  if (V < 0) V = 0;
  const int64_t parts = (dtype == TS_F32) ? ts::kd_parts<float>(V) : ts::kd_parts<ts::bf16_t>(V);
  return 32 + 3 * ts::kd_rows4(n_rows) + (size_t)(n_rows * parts) * sizeof(ts::PartStat);
}

int ts_kdce_fwd_bwd(const void* s, const void* t, const uint8_t* row_mask, const int64_t* labels,
                    int64_t ignore_index, int64_t n_rows, int64_t V, int64_t ld_s, int64_t ld_t, float inv_T,
                    float kd_scale, float ce_weight, void* workspace, float* loss_out, void* grad, int64_t ld_g,
                    int dtype, ts_stream_t stream) {
  // a batch without rows has no logits to point at (its loss is 0/0 = NaN, as the reference gives)
  if (!workspace || !loss_out || (n_rows > 0 && (!s || !t))) return TS_ERR_ARG;
  if (n_rows < 0 || V <= 0 || ld_s < V || ld_t < V || (grad && ld_g < V)) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (!(inv_T > 0.f)) return TS_ERR_ARG;
  // one workgroup (or group of lanes) per row; counts are summed as floats
  if (n_rows > (1 << 24)) return TS_ERR_RANGE;
  const uintptr_t esz = (dtype == TS_F32) ? 4 : 2;
  if (((uintptr_t)s | (uintptr_t)t | (uintptr_t)grad) & (esz - 1)) return TS_ERR_ALIGN;
  if ((uintptr_t)labels & 7u) return TS_ERR_ALIGN;
  if ((uintptr_t)workspace & 31u) return TS_ERR_ALIGN;
  ts::KdArgs a;
  a.s = s;
  a.t = t;
  a.mask = row_mask;
  a.labels = labels;
  a.ignore_index = ignore_index;
  a.n_rows = n_rows;
  a.V = V;
  a.ld_s = ld_s;
  a.ld_t = ld_t;
  a.ld_g = ld_g;
  a.k = inv_T * ts::kLog2e;
  a.kd_gscale = kd_scale * inv_T;
  a.ce_weight = ce_weight;
  a.t_pow = ts::kd_t_pow(inv_T);
  a.counts = nullptr;
  a.self_count = 0;
  a.split_grid = 0;
  a.row_kd = a.row_ce = nullptr;
  a.grad = grad;
  a.n_pieces = 0;
  for (int i = 0; i < ts::kKdMaxPieces; ++i) {
    a.piece_row0[i] = 0;
    a.s_piece[i] = a.t_piece[i] = nullptr;
    a.g_piece[i] = nullptr;
  }
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case TS_F32: return ts::launch_kd<float>(a, kd_scale, workspace, loss_out, st);
    case TS_BF16: return ts::launch_kd<ts::bf16_t>(a, kd_scale, workspace, loss_out, st);
    default: return ts::launch_kd<ts::f16_t>(a, kd_scale, workspace, loss_out, st);
  }
}

int ts_kdce_pieces_fwd_bwd(const void* const* s_pieces, const void* const* t_pieces, void* const* grad_pieces,
                           const int64_t* piece_rows, int n_pieces, const uint8_t* row_mask, const int64_t* labels,
                           int64_t ignore_index, int64_t V, float inv_T, float kd_scale, float ce_weight,
                           void* workspace, float* loss_out, int dtype, ts_stream_t stream) {
  if (!s_pieces || !t_pieces || !piece_rows || !workspace || !loss_out) return TS_ERR_ARG;
  if (n_pieces < 1 || n_pieces > ts::kKdMaxPieces) return TS_ERR_RANGE;
  if (V <= 0 || !(inv_T > 0.f)) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  const uintptr_t esz = (dtype == TS_F32) ? 4 : 2;
  ts::KdArgs a;
  a.s = a.t = nullptr;
  a.grad = nullptr;
  int64_t rows = 0;
  const bool want_grad = grad_pieces && grad_pieces[0];
  for (int i = 0; i < ts::kKdMaxPieces; ++i) {
    a.piece_row0[i] = rows;
    a.s_piece[i] = a.t_piece[i] = nullptr;
    a.g_piece[i] = nullptr;
    if (i >= n_pieces) continue;
    if (piece_rows[i] <= 0 || !s_pieces[i] || !t_pieces[i]) return TS_ERR_ARG;
    if (want_grad != (grad_pieces && grad_pieces[i] != nullptr)) return TS_ERR_ARG;
    void* g = want_grad ? grad_pieces[i] : nullptr;
    if (((uintptr_t)s_pieces[i] | (uintptr_t)t_pieces[i] | (uintptr_t)g) & (esz - 1)) return TS_ERR_ALIGN;
    a.s_piece[i] = s_pieces[i];
    a.t_piece[i] = t_pieces[i];
    a.g_piece[i] = g;
    rows += piece_rows[i];
  }
  if (rows > (1 << 24)) return TS_ERR_RANGE;
  if ((uintptr_t)labels & 7u) return TS_ERR_ALIGN;
  if ((uintptr_t)workspace & 31u) return TS_ERR_ALIGN;
  a.n_pieces = n_pieces;
  a.mask = row_mask;
  a.labels = labels;
  a.ignore_index = ignore_index;
  a.n_rows = rows;
  a.V = V;
  a.ld_s = a.ld_t = a.ld_g = V;
  a.k = inv_T * ts::kLog2e;
  a.kd_gscale = kd_scale * inv_T;
  a.ce_weight = ce_weight;
  a.t_pow = ts::kd_t_pow(inv_T);
  a.counts = nullptr;
  a.self_count = 0;
  a.split_grid = 0;
  a.row_kd = a.row_ce = nullptr;
  hipStream_t st = (hipStream_t)stream;
  switch (dtype) {
    case TS_F32: return ts::launch_kd<float>(a, kd_scale, workspace, loss_out, st);
    case TS_BF16: return ts::launch_kd<ts::bf16_t>(a, kd_scale, workspace, loss_out, st);
    default: return ts::launch_kd<ts::f16_t>(a, kd_scale, workspace, loss_out, st);
  }
}

int ts_kd_fwd_bwd(const void* s, const void* t, const uint8_t* row_mask, int64_t n_rows, int64_t V, int64_t ld_s,
                  int64_t ld_t, float inv_T, float loss_scale, void* workspace, float* loss_out, void* grad,
                  int64_t ld_g, int dtype, ts_stream_t stream) {
  return ts_kdce_fwd_bwd(s, t, row_mask, nullptr, 0, n_rows, V, ld_s, ld_t, inv_T, loss_scale, 0.f, workspace,
                         loss_out, grad, ld_g, dtype, stream);
}

size_t ts_kd_static_scratch_bytes(void) { return ts::kKdStaticScratchBytes; }

int ts_kd_fwd_bwd_static(const void* s, const void* t, const uint8_t* row_mask, int64_t n_rows, int64_t V,
                         int64_t ld_s, int64_t ld_t, float inv_T, float loss_scale, float* loss_out, void* grad,
                         int64_t ld_g, int dtype, ts_stream_t stream) {
  if (n_rows < 0 || V <= 0) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  // the same kernels on the library's own array instead of a caller's workspace
  if (ts_kd_workspace_bytes(n_rows, V, dtype) > ts::kKdStaticScratchBytes) return TS_ERR_RANGE;
  int rc = TS_OK;
  void* ws = ts::kd_static_scratch_ptr(&rc);
  if (!ws) return rc;
  return ts_kdce_fwd_bwd(s, t, row_mask, nullptr, 0, n_rows, V, ld_s, ld_t, inv_T, loss_scale, 0.f, ws, loss_out,
                         grad, ld_g, dtype, stream);
}

}  // extern "C"
