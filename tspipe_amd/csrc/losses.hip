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
  const float rp = fast_exp2(p.m - m), rq = fast_exp2(q.m - m);
  return RowStat{m, p.z * rp + q.z * rq, p.a * rp + q.a * rq};
}

// Reduction over the WIDTH (<= 64, power of two) adjacent lanes of a group.
template <int WIDTH>
__device__ __forceinline__ RowStat stat_lane_reduce(RowStat s) {
#pragma unroll
  for (int off = WIDTH / 2; off > 0; off >>= 1) {
    RowStat o{__shfl_xor(s.m, off, kWave), __shfl_xor(s.z, off, kWave), __shfl_xor(s.a, off, kWave)};
    s = stat_merge(s, o);
  }
  return s;
}

// Folds N (teacher, student) logit pairs into the states.  t, s are the raw
// logits; k = inv_T * log2(e) > 0 scales them into the log2 domain.  The
// block's own maxima are taken first, so each element costs one fma and one
// exp2 per operand, and the running states are rescaled once per block.
template <int N>
__device__ __forceinline__ void stat_block(RowStat& st, RowStat& ss, const float (&t)[N], const float (&s)[N],
                                           float k) {
  float mt = t[0], ms = s[0];
#pragma unroll
  for (int i = 1; i < N; ++i) {
    mt = fmaxf(mt, t[i]);
    ms = fmaxf(ms, s[i]);
  }
  const float mtk = mt * k, msk = ms * k;
  float zt = 0.f, at = 0.f, zs = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float et = fast_exp2(fmaf(t[i], k, -mtk));
    zt += et;
    at = fmaf(et, t[i] - s[i], at);
    zs += fast_exp2(fmaf(s[i], k, -msk));
  }
  st = stat_merge(st, RowStat{mtk, zt, at * k});
  ss = stat_merge(ss, RowStat{msk, zs, 0.f});
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

// One group of GROUP threads per row; BLOCK/GROUP rows per workgroup.  GROUP
// is 16, 32 or 64 lanes of a wavefront for narrow rows, or the whole
// workgroup (GROUP == BLOCK) for wide ones.
//   pass 1: one sweep over both rows -> (max, sum-exp, weighted sum) of the
//           teacher row and (max, sum-exp) of the student row, online.
//   pass 2: grad = g * (q - p).
// KREG > 0: the row pair is held in registers between the passes (KREG
// 16-byte vectors per thread and operand, all loads issued up front), so
// each logit is read from memory once; the launcher guarantees
// ceil(V / VEC) <= KREG * GROUP.  KREG == 0: any width, pass 2 re-reads the
// rows (they are L2-resident: the group has just read them).
// Rows with mask == 0 only zero their gradient row.
template <typename T, int BLOCK, int GROUP, int KREG>
__global__ __launch_bounds__(BLOCK) void kd_rows_kernel(
    const T* __restrict__ s, const T* __restrict__ t, const uint8_t* __restrict__ mask,
    const int* __restrict__ n_sel_dev, int64_t n_rows, int64_t V, int64_t ld_s, int64_t ld_t,
    int64_t ld_g, float kscale /* inv_T * log2(e) */, float gscale /* loss_scale * inv_T */,
    float* __restrict__ row_loss, T* __restrict__ grad) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int NW = GROUP / kWave;  // wavefronts per group (0 for sub-wavefront groups)
  constexpr int KR = KREG > 0 ? KREG : 1;
  __shared__ RowStat lds_t[BLOCK / kWave];
  __shared__ RowStat lds_s[BLOCK / kWave];

  const int gtid = threadIdx.x % GROUP;
  const int64_t row = (int64_t)blockIdx.x * (BLOCK / GROUP) + threadIdx.x / GROUP;
  // With GROUP == BLOCK the whole workgroup shares one row, so the early
  // exits below are uniform; smaller groups never reach a __syncthreads and
  // only shuffle among their own lanes.
  if (row >= n_rows) return;

  const T* srow = s + row * ld_s;
  const T* trow = t + row * ld_t;
  T* grow = grad ? grad + row * ld_g : nullptr;

  const bool selected = mask ? (mask[row] != 0) : true;

  // Common misalignment of the three rows: `head` elements come before the
  // first 16-byte boundary.  If the rows disagree everything is "head" and
  // goes through the scalar path.
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

  Vec16<T> rt[KR], rs[KR];
  if (KREG > 0) {
#pragma unroll
    for (int j = 0; j < KR; ++j) {
      const int64_t v = gtid + (int64_t)j * GROUP;
      if (v < nvec) {
        rt[j] = load16(trow + head + v * VEC);
        rs[j] = load16(srow + head + v * VEC);
      }
    }
  }

  RowStat st = stat_init(), ss = stat_init();
  {
    float xt1[1], xs1[1];
    for (int64_t i = gtid; i < head; i += GROUP) {
      xt1[0] = to_f32(trow[i]);
      xs1[0] = to_f32(srow[i]);
      stat_block<1>(st, ss, xt1, xs1, kscale);
    }
    for (int64_t i = tail0 + gtid; i < V; i += GROUP) {
      xt1[0] = to_f32(trow[i]);
      xs1[0] = to_f32(srow[i]);
      stat_block<1>(st, ss, xt1, xs1, kscale);
    }
    float xt[VEC], xs[VEC];
    if (KREG > 0) {
#pragma unroll
      for (int j = 0; j < KR; ++j) {
        if (gtid + (int64_t)j * GROUP < nvec) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            xt[i] = to_f32(rt[j].v[i]);
            xs[i] = to_f32(rs[j].v[i]);
          }
          stat_block<VEC>(st, ss, xt, xs, kscale);
        }
      }
    } else {
      for (int64_t v = gtid; v < nvec; v += GROUP) {
        const Vec16<T> vt = load16(trow + head + v * VEC);
        const Vec16<T> vs = load16(srow + head + v * VEC);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          xt[i] = to_f32(vt.v[i]);
          xs[i] = to_f32(vs.v[i]);
        }
        stat_block<VEC>(st, ss, xt, xs, kscale);
      }
    }
  }

  st = stat_lane_reduce<(GROUP < kWave ? GROUP : kWave)>(st);
  ss = stat_lane_reduce<(GROUP < kWave ? GROUP : kWave)>(ss);
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
    const float p = fast_exp2(fmaf(to_f32(trow[i]), kscale, -lse_t));
    const float q = fast_exp2(fmaf(to_f32(srow[i]), kscale, -lse_s));
    grow[i] = from_f32<T>(g * (q - p));
  }
  for (int64_t i = tail0 + gtid; i < V; i += GROUP) {
    const float p = fast_exp2(fmaf(to_f32(trow[i]), kscale, -lse_t));
    const float q = fast_exp2(fmaf(to_f32(srow[i]), kscale, -lse_s));
    grow[i] = from_f32<T>(g * (q - p));
  }
  if (KREG > 0) {
#pragma unroll
    for (int j = 0; j < KR; ++j) {
      const int64_t v = gtid + (int64_t)j * GROUP;
      if (v < nvec) {
        Vec16<T> o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const float p = fast_exp2(fmaf(to_f32(rt[j].v[i]), kscale, -lse_t));
          const float q = fast_exp2(fmaf(to_f32(rs[j].v[i]), kscale, -lse_s));
          o.v[i] = from_f32<T>(g * (q - p));
        }
        store16(grow + head + v * VEC, o);
      }
    }
  } else {
    for (int64_t v = gtid; v < nvec; v += GROUP) {
      const Vec16<T> vt = load16(trow + head + v * VEC);
      const Vec16<T> vs = load16(srow + head + v * VEC);
      Vec16<T> o;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float p = fast_exp2(fmaf(to_f32(vt.v[i]), kscale, -lse_t));
        const float q = fast_exp2(fmaf(to_f32(vs.v[i]), kscale, -lse_s));
        o.v[i] = from_f32<T>(g * (q - p));
      }
      store16(grow + head + v * VEC, o);
    }
  }
}

// ---- wide rows: a row is cut into parts of kPartVecs 16-byte vectors, one
// short-lived 256-thread workgroup per (row, part), two launches:
//   pass 1, grid = every (row, part): selected rows -> partial online-softmax
//           state of the part (part_stats[row][part]); unselected rows ->
//           zero-fill of the part's gradient.  The first kind is bound by
//           exp2 throughput, the second by HBM writes, and they overlap.
//   pass 2, bounded grid walking the (selected row, part) items of the
//           compacted row list: merges the row's partial states, writes the
//           part's gradient.  Its reads come out of the 256 MB last-level
//           cache when the selected rows fit there.
// Every workgroup issues its loads up front and is short-lived, which is the
// shape that streams best on this GPU, and rows spread evenly over the CUs
// whatever the mask looks like.
constexpr int kPartBlock = 256;
constexpr int kPartPerThread = 4;
constexpr int kPartVecs = kPartBlock * kPartPerThread;
constexpr int kPass2MaxGrid = 8192;

struct RowGeom {
  int64_t head, nvec, tail0;
};

// Split of a row by the common 16-byte misalignment of s and t (all scalar
// when they disagree).
template <typename T>
__device__ __forceinline__ RowGeom row_geom(const T* srow, const T* trow, int64_t V) {
  constexpr int VEC = Vec16<T>::N;
  const uint32_t mis_s = (uint32_t)((uintptr_t)srow & 15u), mis_t = (uint32_t)((uintptr_t)trow & 15u);
  RowGeom g;
  g.head = (mis_s == mis_t) ? (int64_t)(((16u - mis_s) & 15u) / sizeof(T)) : V;
  if (g.head > V) g.head = V;
  g.nvec = (V - g.head) / VEC;
  g.tail0 = g.head + g.nvec * VEC;
  return g;
}

struct PartStat {  // 32 bytes
  float mt, zt, at, ms, zs, pad0, pad1, pad2;
};

template <typename T>
__global__ __launch_bounds__(kPartBlock) void kd_wide_pass1_kernel(
    const T* __restrict__ s, const T* __restrict__ t, const uint8_t* __restrict__ mask, int64_t V,
    int64_t ld_s, int64_t ld_t, int64_t ld_g, int parts, float kscale, PartStat* __restrict__ part_stats,
    float* __restrict__ row_loss, T* __restrict__ grad) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ RowStat lds_t[kPartBlock / kWave];
  __shared__ RowStat lds_s[kPartBlock / kWave];
  const int64_t row = blockIdx.x / parts;
  const int part = (int)(blockIdx.x % parts);
  const int tid = threadIdx.x;
  const int64_t v0 = (int64_t)part * kPartVecs;

  if (mask && mask[row] == 0) {
    if (part == 0 && tid == 0) row_loss[row] = 0.f;
    if (!grad) return;
    T* grow = grad + row * ld_g;
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
    return;
  }

  const T* srow = s + row * ld_s;
  const T* trow = t + row * ld_t;
  const RowGeom g = row_geom<T>(srow, trow, V);
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
  RowStat st = stat_init(), ss = stat_init();
  float xt1[1], xs1[1];
  if (part == 0) {
    for (int64_t i = tid; i < g.head; i += kPartBlock) {
      xt1[0] = to_f32(trow[i]);
      xs1[0] = to_f32(srow[i]);
      stat_block<1>(st, ss, xt1, xs1, kscale);
    }
  }
  if (part == parts - 1) {
    for (int64_t i = g.tail0 + tid; i < V; i += kPartBlock) {
      xt1[0] = to_f32(trow[i]);
      xs1[0] = to_f32(srow[i]);
      stat_block<1>(st, ss, xt1, xs1, kscale);
    }
  }
  // Vector body.  The maximum is settled first, over the thread's vectors and
  // then across the wavefront, so that every lane exponentiates against the
  // same reference and the sums combine by plain addition: 2 exp2 per pair
  // and no per-step rescaling.
  float mt = st.m, ms = ss.m;  // scaled domain (kNegBig when the thread had no ragged element)
  float ft[kPartPerThread][VEC], fs[kPartPerThread][VEC];
#pragma unroll
  for (int j = 0; j < kPartPerThread; ++j) {
    if (v0 + tid + j * kPartBlock < g.nvec) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        ft[j][i] = to_f32(rt[j].v[i]);
        fs[j][i] = to_f32(rs[j].v[i]);
        mt = fmaxf(mt, ft[j][i] * kscale);
        ms = fmaxf(ms, fs[j][i] * kscale);
      }
    }
  }
  const float wmt = wave_max(mt), wms = wave_max(ms);
  // ragged-end sums re-based onto the wavefront's maxima
  float zt = st.z * fast_exp2(st.m - wmt), at = st.a * fast_exp2(st.m - wmt);
  float zs = ss.z * fast_exp2(ss.m - wms);
  float araw = 0.f;  // sum e_t * (t - s) over the vector body, raw logit units
#pragma unroll
  for (int j = 0; j < kPartPerThread; ++j) {
    if (v0 + tid + j * kPartBlock < g.nvec) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float et = fast_exp2(fmaf(ft[j][i], kscale, -wmt));
        zt += et;
        araw = fmaf(et, ft[j][i] - fs[j][i], araw);
        zs += fast_exp2(fmaf(fs[j][i], kscale, -wms));
      }
    }
  }
  at = fmaf(araw, kscale, at);
  zt = wave_sum(zt);
  at = wave_sum(at);
  zs = wave_sum(zs);
  const int w = tid / kWave, lane = tid % kWave;
  if (lane == 0) {
    lds_t[w] = RowStat{wmt, zt, at};
    lds_s[w] = RowStat{wms, zs, 0.f};
  }
  __syncthreads();
  if (tid == 0) {
    RowStat bt = lds_t[0], bs = lds_s[0];
#pragma unroll
    for (int i = 1; i < kPartBlock / kWave; ++i) {
      bt = stat_merge(bt, lds_t[i]);
      bs = stat_merge(bs, lds_s[i]);
    }
    part_stats[row * parts + part] = PartStat{bt.m, bt.z, bt.a, bs.m, bs.z, 0.f, 0.f, 0.f};
  }
}

template <typename T>
__global__ __launch_bounds__(kPartBlock) void kd_wide_pass2_kernel(
    const T* __restrict__ s, const T* __restrict__ t, const int* __restrict__ sel_rows,
    const int* __restrict__ n_sel_dev, int64_t n_rows, int64_t V, int64_t ld_s, int64_t ld_t, int64_t ld_g,
    int parts, float kscale, float gscale, const PartStat* __restrict__ part_stats,
    float* __restrict__ row_loss, T* __restrict__ grad) {
  constexpr int VEC = Vec16<T>::N;
  const int64_t n_sel = n_sel_dev ? (int64_t)(*n_sel_dev) : n_rows;
  const int64_t items = n_sel * parts;
  const int tid = threadIdx.x;
  const float gg = gscale / (float)n_sel;

  for (int64_t item = blockIdx.x; item < items; item += gridDim.x) {
    const int64_t row = sel_rows ? (int64_t)sel_rows[item / parts] : item / parts;
    const int part = (int)(item % parts);
    const int64_t v0 = (int64_t)part * kPartVecs;
    const T* srow = s + row * ld_s;
    const T* trow = t + row * ld_t;
    T* grow = grad ? grad + row * ld_g : nullptr;
    const RowGeom g = row_geom<T>(srow, trow, V);
    const bool gvec = grow && (((uintptr_t)grow & 15u) == ((uintptr_t)srow & 15u));

    Vec16<T> rt[kPartPerThread], rs[kPartPerThread];
    if (grow) {
#pragma unroll
      for (int j = 0; j < kPartPerThread; ++j) {
        const int64_t v = v0 + tid + j * kPartBlock;
        if (v < g.nvec) {
          rt[j] = load16(trow + g.head + v * VEC);
          rs[j] = load16(srow + g.head + v * VEC);
        }
      }
    }
    // every thread merges the row's few partial states itself (uniform loads)
    RowStat st = stat_init(), ss = stat_init();
    for (int p = 0; p < parts; ++p) {
      const PartStat ps = part_stats[row * parts + p];
      st = stat_merge(st, RowStat{ps.mt, ps.zt, ps.at});
      ss = stat_merge(ss, RowStat{ps.ms, ps.zs, 0.f});
    }
    const float lse_t = st.m + log2f(st.z);
    const float lse_s = ss.m + log2f(ss.z);
    if (part == 0 && tid == 0) row_loss[row] = kLn2 * (st.a / st.z - lse_t + lse_s);
    if (!grow) continue;
    auto one = [&](T tv, T sv) {
      const float p = fast_exp2(fmaf(to_f32(tv), kscale, -lse_t));
      const float q = fast_exp2(fmaf(to_f32(sv), kscale, -lse_s));
      return from_f32<T>(gg * (q - p));
    };
    if (part == 0)
      for (int64_t i = tid; i < g.head; i += kPartBlock) grow[i] = one(trow[i], srow[i]);
    if (part == parts - 1)
      for (int64_t i = g.tail0 + tid; i < V; i += kPartBlock) grow[i] = one(trow[i], srow[i]);
#pragma unroll
    for (int j = 0; j < kPartPerThread; ++j) {
      const int64_t v = v0 + tid + j * kPartBlock;
      if (v < g.nvec) {
        Vec16<T> o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) o.v[i] = one(rt[j].v[i], rs[j].v[i]);
        if (gvec) {
          store16(grow + g.head + v * VEC, o);
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) grow[g.head + v * VEC + i] = o.v[i];
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

// n_sel = number of non-zero mask bytes and, when sel_rows is given, the
// indices of those rows in ascending order.  One workgroup; thread i owns the
// i-th contiguous slice of the mask.
__global__ __launch_bounds__(1024) void mask_count_kernel(const uint8_t* __restrict__ mask, int64_t n,
                                                          int* __restrict__ out, int* __restrict__ sel_rows) {
  __shared__ int scan[1024];
  const int tid = threadIdx.x;
  const int64_t per = (n + 1023) / 1024;
  const int64_t lo = tid * per, hi = (lo + per < n) ? lo + per : n;
  int c = 0;
  for (int64_t i = lo; i < hi; ++i) c += mask[i] != 0;
  scan[tid] = c;
  __syncthreads();
  // inclusive Hillis-Steele scan over the 1024 per-thread counts
  for (int off = 1; off < 1024; off <<= 1) {
    const int add = (tid >= off) ? scan[tid - off] : 0;
    __syncthreads();
    scan[tid] += add;
    __syncthreads();
  }
  if (tid == 1023) *out = scan[1023];
  if (sel_rows) {
    int pos = scan[tid] - c;
    for (int64_t i = lo; i < hi; ++i)
      if (mask[i] != 0) sel_rows[pos++] = (int)i;
  }
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
  // workspace (see ts_kd_workspace_bytes): [0,32) selected-row count;
  // row_loss[n_rows]; sel_rows[n_rows]; then the partial states of the
  // wide-row path; every region 32-byte aligned
  const int64_t parts = kd_parts<T>(V);
  const size_t rows4 = (size_t)((n_rows * 4 + 31) / 32) * 32;
  char* wsb = reinterpret_cast<char*>(ws);
  int* n_sel = reinterpret_cast<int*>(wsb);
  float* row_loss = reinterpret_cast<float*>(wsb + 32);
  int* sel_rows = reinterpret_cast<int*>(wsb + 32 + rows4);
  PartStat* part_stats = reinterpret_cast<PartStat*>(wsb + 32 + 2 * rows4);
  if (mask) {
    hipLaunchKernelGGL(mask_count_kernel, dim3(1), dim3(1024), 0, stream, mask, n_rows, n_sel,
                       parts ? sel_rows : (int*)nullptr);
    int rc = check_launch();
    if (rc) return rc;
  }
  const int* n_sel_arg = mask ? n_sel : nullptr;
  const float kscale = inv_T * kLog2e, gscale = loss_scale * inv_T;
  const T* sp = reinterpret_cast<const T*>(s);
  const T* tp = reinterpret_cast<const T*>(t);
  T* gp = reinterpret_cast<T*>(grad);
  // 16-byte vectors a row can span, counting a ragged first and last one
  const int64_t vecs = (V + Vec16<T>::N - 1) / Vec16<T>::N + 1;
#define TS_KD_LAUNCH(BLOCK, GROUP, KREG)                                                                  \
  hipLaunchKernelGGL((kd_rows_kernel<T, BLOCK, GROUP, KREG>),                                             \
                     dim3((unsigned)((n_rows + (BLOCK / GROUP) - 1) / (BLOCK / GROUP))), dim3(BLOCK), 0,  \
                     stream, sp, tp, mask, n_sel_arg, n_rows, V, ld_s, ld_t, ld_g, kscale, gscale,        \
                     row_loss, gp)
  if (vecs <= 16 * 2) {
    TS_KD_LAUNCH(256, 16, 2);
  } else if (vecs <= 32 * 2) {
    TS_KD_LAUNCH(256, 32, 2);
  } else if (vecs <= 64 * 4) {
    TS_KD_LAUNCH(256, 64, 4);
  } else if (parts == 0) {
    TS_KD_LAUNCH(256, 256, 4);
  } else {
    const int64_t items = n_rows * parts;
    if (items > 0x7fffffffLL) return TS_ERR_RANGE;
    hipLaunchKernelGGL((kd_wide_pass1_kernel<T>), dim3((unsigned)items), dim3(kPartBlock), 0, stream, sp, tp,
                       mask, V, ld_s, ld_t, ld_g, (int)parts, kscale, part_stats, row_loss, gp);
    int rc = check_launch();
    if (rc) return rc;
    const int64_t grid2 = items < kPass2MaxGrid ? items : kPass2MaxGrid;
    hipLaunchKernelGGL((kd_wide_pass2_kernel<T>), dim3((unsigned)grid2), dim3(kPartBlock), 0, stream, sp, tp,
                       mask ? sel_rows : (const int*)nullptr, n_sel_arg, n_rows, V, ld_s, ld_t, ld_g, (int)parts,
                       kscale, gscale, part_stats, row_loss, gp);
  }
#undef TS_KD_LAUNCH
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

size_t ts_kd_workspace_bytes(int64_t n_rows, int64_t V, int dtype) {
  if (n_rows < 0) n_rows = 0;
  if (V < 0) V = 0;
  const int64_t parts = (dtype == TS_F32) ? ts::kd_parts<float>(V) : ts::kd_parts<ts::bf16_t>(V);
  return (size_t)(32 + 2 * (((n_rows * 4 + 31) / 32) * 32) + n_rows * parts * (int64_t)sizeof(ts::PartStat));
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
  if ((uintptr_t)workspace & 31u) return TS_ERR_ALIGN;
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
