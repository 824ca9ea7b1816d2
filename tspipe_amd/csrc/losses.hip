// Row-wise losses with fused backward (BYOL normalised MSE and cosine embedding
// on embedding-sized rows, one 64-wide wavefront per row; squared error
// between logits) and the small shared reductions.  All accumulation is fp32; storage is fp32, bf16 or
// fp16.
#include "common.h"

namespace ts {

// out = scale * sum(v[0..n)) / denom, summed in a fixed order (deterministic).
__global__ __launch_bounds__(1024) void sum_scale_kernel(const float* __restrict__ v, int64_t n,
                                                         float scale, const int* __restrict__ denom_dev,
                                                         float denom, float* __restrict__ out) {
  __shared__ float lds[1024 / kWave];
  const float tot = block_sum<1024 / kWave>(thread_share_of_sum<1024>(v, n), lds);
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
// The operands of both (x, y) pairs as up to kByolMaxPieces row blocks each
// (micro-batch outputs that were never concatenated): piece i holds rows
// row0[i] .. row0[i+1]-1.  A single matrix is one piece.
constexpr int kByolMaxPieces = 8;
struct ByolArgs {
  int n_pieces;
  int64_t row0[kByolMaxPieces];
  const void* x[2][kByolMaxPieces];
  const void* y[2][kByolMaxPieces];
  void* g[2][kByolMaxPieces];  // per pair: all null or all set
};

// One wavefront per (pair, row).  x^ = x / max(|x|, eps) as F.normalize does.
template <typename T>
__global__ __launch_bounds__(256) void byol_rows_kernel(const ByolArgs args, int pairs, int64_t n, int64_t c,
                                                        float* __restrict__ row_loss) {
  constexpr float kEps = 1e-12f;
  const int lane = threadIdx.x % kWave;
  const int64_t vrow = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  const int64_t total = pairs * n;
  if (vrow >= total) return;
  const int second = vrow >= n ? 1 : 0;
  const int64_t row = second ? vrow - n : vrow;
  // the piece is found with a chain of selects (uniform per wavefront)
  const void* xb = args.x[second][0];
  const void* yb = args.y[second][0];
  void* gb = args.g[second][0];
  int64_t r0 = 0;
#pragma unroll
  for (int i = 1; i < kByolMaxPieces; ++i) {
    const bool ge = i < args.n_pieces && row >= args.row0[i];
    xb = ge ? args.x[second][i] : xb;
    yb = ge ? args.y[second][i] : yb;
    gb = ge ? args.g[second][i] : gb;
    r0 = ge ? args.row0[i] : r0;
  }
  const T* x = (const T*)xb + (row - r0) * c;
  const T* y = (const T*)yb + (row - r0) * c;
  T* gx = gb ? (T*)gb + (row - r0) * c : nullptr;

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


// n_sel = number of non-zero mask bytes.  One workgroup.
__global__ __launch_bounds__(1024) void mask_count_kernel(const uint8_t* __restrict__ mask, int64_t n,
                                                          int* __restrict__ out) {
  __shared__ float lds[1024 / kWave];
  const float tot = mask_count_block<1024>(mask, n, lds);  // exact in float for any n the launchers accept
  if (threadIdx.x == 0) *out = (int)tot;
}

// Two row-wise operands and an optional gradient as up to kRowMaxPieces row
// blocks each (micro-batch outputs that were never concatenated): piece i
// holds rows row0[i] .. row0[i+1]-1, contiguous rows of the common width.
// n_pieces == 0 means the single matrices a / b / g with leading dimensions.
constexpr int kRowMaxPieces = 8;
struct RowPieces {
  const void* a;
  const void* b;
  void* g;
  int64_t ld_a, ld_b, ld_g;
  int n_pieces;
  int64_t row0[kRowMaxPieces];
  const void* ap[kRowMaxPieces];
  const void* bp[kRowMaxPieces];
  void* gp[kRowMaxPieces];  // all null or all set
};

template <typename T>
struct RowPtrs {
  const T* a;
  const T* b;
  T* g;
};

// Pointers to one batch row (the piece is found with a chain of selects,
// uniform for a wavefront or workgroup that shares a row).
template <typename T>
__device__ __forceinline__ RowPtrs<T> row_ptrs(const RowPieces& t, int64_t row) {
  RowPtrs<T> r;
  if (t.n_pieces == 0) {
    r.a = (const T*)t.a + row * t.ld_a;
    r.b = (const T*)t.b + row * t.ld_b;
    r.g = t.g ? (T*)t.g + row * t.ld_g : nullptr;
    return r;
  }
  const void* ab = t.ap[0];
  const void* bb = t.bp[0];
  void* gb = t.gp[0];
  int64_t r0 = 0;
#pragma unroll
  for (int i = 1; i < kRowMaxPieces; ++i) {
    const bool ge = i < t.n_pieces && row >= t.row0[i];
    ab = ge ? t.ap[i] : ab;
    bb = ge ? t.bp[i] : bb;
    gb = ge ? t.gp[i] : gb;
    r0 = ge ? t.row0[i] : r0;
  }
  const int64_t local = row - r0;
  r.a = (const T*)ab + local * t.ld_a;
  r.b = (const T*)bb + local * t.ld_b;
  r.g = gb ? (T*)gb + local * t.ld_g : nullptr;
  return r;
}

inline RowPieces row_single(const void* a, const void* b, void* g, int64_t ld_a, int64_t ld_b, int64_t ld_g) {
  RowPieces t;
  t.a = a;
  t.b = b;
  t.g = g;
  t.ld_a = ld_a;
  t.ld_b = ld_b;
  t.ld_g = ld_g;
  t.n_pieces = 0;
  for (int i = 0; i < kRowMaxPieces; ++i) {
    t.row0[i] = 0;
    t.ap[i] = t.bp[i] = nullptr;
    t.gp[i] = nullptr;
  }
  return t;
}

// Fills a piece table from host arrays of device pointers; returns a status
// and the total number of rows.
inline int row_pieces(const void* const* a, const void* const* b, void* const* g, const int64_t* piece_rows,
                      int n_pieces, int64_t width, size_t elem, RowPieces* out, int64_t* total) {
  if (!a || !b || !piece_rows) return TS_ERR_ARG;
  if (n_pieces < 1 || n_pieces > kRowMaxPieces) return TS_ERR_RANGE;
  RowPieces t = row_single(nullptr, nullptr, nullptr, width, width, width);
  const bool want = g && g[0];
  int64_t rows = 0;
  for (int i = 0; i < n_pieces; ++i) {
    if (piece_rows[i] <= 0 || !a[i] || !b[i]) return TS_ERR_ARG;
    if (want != (g && g[i] != nullptr)) return TS_ERR_ARG;
    if (((uintptr_t)a[i] | (uintptr_t)b[i] | (uintptr_t)(want ? g[i] : nullptr)) & (elem - 1)) return TS_ERR_ALIGN;
    t.row0[i] = rows;
    t.ap[i] = a[i];
    t.bp[i] = b[i];
    t.gp[i] = want ? g[i] : nullptr;
    rows += piece_rows[i];
  }
  t.n_pieces = n_pieces;
  *out = t;
  *total = rows;
  return TS_OK;
}

// ---- cosine embedding loss with target +1 ----------------------------------
//   cos_i = <x_i, y_i> / sqrt((|x_i|^2 + eps)(|y_i|^2 + eps)),  eps = 1e-12
//   loss  = weight * mean over selected rows of (1 - cos_i);  gradient to x only.
template <typename T>
__global__ __launch_bounds__(256) void cosine_rows_kernel(const RowPieces tab, const uint8_t* __restrict__ mask,
                                                          int64_t n, int64_t c, float weight,
                                                          float* __restrict__ row_loss) {
  constexpr float kEps = 1e-12f;
  __shared__ float lds_cnt[256 / kWave];
  // the number of selected rows scales the gradient: every workgroup counts the
  // mask's few kilobytes itself (no counting launch in front)
  const float n_sel = mask ? mask_count_block<256>(mask, n, lds_cnt) : (float)n;
  const int lane = threadIdx.x % kWave;
  const int64_t row = (int64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
  if (row >= n) return;
  const RowPtrs<T> rp = row_ptrs<T>(tab, row);
  const T* xr = rp.a;
  const T* yr = rp.b;
  T* gr = rp.g;
  if (mask && mask[row] == 0) {
    if (lane == 0) row_loss[row] = 0.f;
    if (gr)
      for (int64_t i = lane; i < c; i += kWave) gr[i] = from_f32<T>(0.f);
    return;
  }
  float sxx = 0.f, syy = 0.f, sxy = 0.f;
  for (int64_t i = lane; i < c; i += kWave) {
    const float a = to_f32(xr[i]), b = to_f32(yr[i]);
    sxx += a * a;
    syy += b * b;
    sxy += a * b;
  }
  sxx = wave_sum(sxx) + kEps;
  syy = wave_sum(syy) + kEps;
  sxy = wave_sum(sxy);
  const float inv_den = 1.f / sqrtf(sxx * syy);
  const float cosv = sxy * inv_den;
  if (lane == 0) row_loss[row] = 1.f - cosv;
  if (!gr) return;
  const float k = -weight / n_sel;
  const float proj = cosv / sxx;
  for (int64_t i = lane; i < c; i += kWave) {
    const float a = to_f32(xr[i]), b = to_f32(yr[i]);
    gr[i] = from_f32<T>(k * (b * inv_den - proj * a));
  }
}

// loss = weight * sum(row_loss) / selected rows, fixed summation order; the
// workgroup counts the mask itself.  0/0 = NaN for an empty selection, as the
// reference gives.
__global__ __launch_bounds__(1024) void cosine_finalize_kernel(const float* __restrict__ row_loss, int64_t n,
                                                               float weight, const uint8_t* __restrict__ mask,
                                                               float* __restrict__ out) {
  __shared__ float lds[1024 / kWave];
  const float n_sel = mask ? mask_count_block<1024>(mask, n, lds) : (float)n;
  const float tot = block_sum<1024 / kWave>(thread_share_of_sum<1024>(row_loss, n), lds);
  if (threadIdx.x == 0) *out = weight * (tot / n_sel);
}

// ---- squared error between logits (fused backward) -----------------------
//   loss = weight * sum over selected rows, all columns of (s - t)^2 / denom
//   grad = d loss / d s = (2 weight / denom)(s - t) on selected rows, 0 elsewhere
// denom = selected rows (x V when the mean runs over elements).  Every row
// leaves one partial sum; a last single-workgroup launch adds them in a fixed
// order.
// Rows below kMseLongMin elements: GROUP lanes of a wavefront own a row (16
// lanes for rows of up to 32 16-byte vectors, a whole wavefront beyond), four
// wavefronts to a workgroup, no LDS and no barrier: each lane keeps up to four
// vectors per operand in flight, the row's sum is a shuffle reduction.
// 32768 x 1000 fp32, us per call without a mask / under a 15 % mask: 71 / 49
// against 115 / 110 for the form this replaces (a 256-thread workgroup per
// 4096 elements of a row with a block reduction: 250 of 1024 vector slots used
// at that width).  kMseSpan only sizes the workspace now.
constexpr int kMseBlock = 256;
constexpr int kMseSpan = 4096;
constexpr int kMseShortRegs = 4;

// One element: its squared difference into acc, its gradient (or a zero) out.
template <typename T>
__device__ __forceinline__ T mse_grad_one(T sv, T tv, T gold, float k, int accumulate, float& acc) {
  const float d = to_f32(sv) - to_f32(tv);
  acc += d * d;
  return from_f32<T>(accumulate ? to_f32(gold) + k * d : k * d);
}

template <typename T, int GROUP, bool ACC>
__global__ __launch_bounds__(kMseBlock) void mse_rows_kernel(const RowPieces tab, const uint8_t* __restrict__ mask,
                                                              const int* __restrict__ n_sel_dev, int64_t n_rows,
                                                              int64_t V, float weight, int per_element,
                                                              float* __restrict__ partial) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int accumulate = ACC ? 1 : 0;
  const int gtid = threadIdx.x % GROUP;
  const int64_t row = (int64_t)blockIdx.x * (kMseBlock / GROUP) + threadIdx.x / GROUP;
  if (row >= n_rows) return;  // whole groups leave together; nothing below synchronises across groups
  const bool sel = !mask || mask[row] != 0;
  const RowPtrs<T> rp = row_ptrs<T>(tab, row);
  const T* sr = rp.a;
  const T* tr = rp.b;
  T* gr = rp.g;
  const T zero = from_f32<T>(0.f);
  if (!sel) {
    if (gtid == 0) partial[row] = 0.f;
    if (!gr || ACC) return;
    const uint32_t mis = (uint32_t)((uintptr_t)gr & 15u);
    int64_t head = (int64_t)(((16u - mis) & 15u) / sizeof(T));
    if (head > V) head = V;
    const int64_t nvec = (V - head) / VEC, tail0 = head + nvec * VEC;
    Vec16<T> z;
#pragma unroll
    for (int e = 0; e < VEC; ++e) z.v[e] = zero;
    if (gtid < head) gr[gtid] = zero;
    for (int64_t v = gtid; v < nvec; v += GROUP) store16(gr + head + v * VEC, z);  // plain stores: a zero-fill
    if (tail0 + gtid < V) gr[tail0 + gtid] = zero;
    return;
  }
  const float rows_sel = n_sel_dev ? (float)(*n_sel_dev) : (float)n_rows;
  const float k = 2.f * weight / (per_element ? rows_sel * (float)V : rows_sel);
  const uint32_t mis = (uint32_t)((uintptr_t)sr & 15u);
  const bool alike = mis == (uint32_t)((uintptr_t)tr & 15u) && (!gr || mis == (uint32_t)((uintptr_t)gr & 15u)) &&
                     mis % sizeof(T) == 0;
  int64_t head = alike ? (int64_t)(((16u - mis) & 15u) / sizeof(T)) : V;
  if (head > V) head = V;
  const int64_t nvec = (V - head) / VEC, tail0 = head + nvec * VEC;
  const bool acc_g = gr && ACC;
  float acc = 0.f;
  // the few elements in front of and behind the row's aligned middle (all of the row when the operands
  // are aligned differently)
  for (int64_t i = gtid; i < head; i += GROUP) {
    const T gv = mse_grad_one<T>(sr[i], tr[i], acc_g ? gr[i] : zero, k, accumulate, acc);
    if (gr) gr[i] = gv;
  }
  if (tail0 + gtid < V) {
    const int64_t i = tail0 + gtid;
    const T gv = mse_grad_one<T>(sr[i], tr[i], acc_g ? gr[i] : zero, k, accumulate, acc);
    if (gr) gr[i] = gv;
  }
  const T* s4 = sr + head;
  const T* t4 = tr + head;
  T* g4 = gr + head;
  for (int64_t base = 0; base < nvec; base += (int64_t)GROUP * kMseShortRegs) {
    Vec16<T> vs[kMseShortRegs], vt[kMseShortRegs], vg[ACC ? kMseShortRegs : 1];
#pragma unroll
    for (int j = 0; j < kMseShortRegs; ++j) {
      const int64_t v = base + gtid + (int64_t)j * GROUP;
      if (v < nvec) {
        vs[j] = load16_stream(s4 + v * VEC);  // read once
        vt[j] = load16_stream(t4 + v * VEC);
        if (acc_g) vg[ACC ? j : 0] = load16(g4 + v * VEC);
      }
    }
#pragma unroll
    for (int j = 0; j < kMseShortRegs; ++j) {
      const int64_t v = base + gtid + (int64_t)j * GROUP;
      if (v < nvec) {
        Vec16<T> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          o.v[e] = mse_grad_one<T>(vs[j].v[e], vt[j].v[e], acc_g ? vg[ACC ? j : 0].v[e] : zero, k, accumulate, acc);
        if (gr) {
          if (ACC)
            store16(g4 + v * VEC, o);
          else
            store16_stream(g4 + v * VEC, o);
        }
      }
    }
  }
#pragma unroll
  for (int off = GROUP / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, kWave);
  if (gtid == 0) partial[row] = acc;
}

// out (+)= weight * sum(partial) / denom, fixed summation order
__global__ __launch_bounds__(1024) void mse_finalize_kernel(const float* __restrict__ partial, int64_t n,
                                                            const int* __restrict__ n_sel_dev,
                                                            const uint8_t* __restrict__ mask, int64_t n_rows,
                                                            int64_t V, float weight, int per_element, int accumulate,
                                                            float* __restrict__ out) {
  __shared__ float lds[1024 / kWave];
  // no counting launch ran in front (the long-row route): the selected rows are counted here
  const float counted = (!n_sel_dev && mask) ? mask_count_block<1024>(mask, n_rows, lds) : (float)n_rows;
  const float tot = block_sum<1024 / kWave>(thread_share_of_sum<1024>(partial, n), lds);
  if (threadIdx.x == 0) {
    const float rows_sel = n_sel_dev ? (float)(*n_sel_dev) : counted;
    const float denom = per_element ? rows_sel * (float)V : rows_sel;
    const float v = weight * (tot / denom);  // 0/0 = NaN for an empty selection, as the reference gives
    *out = accumulate ? *out + v : v;
  }
}

// Rows of at least kMseLongMin elements: one 512-thread workgroup per row, all
// of a row's loads issued up front (up to kMseLongRegs 16-byte vectors per
// thread and operand at a time; longer rows in rounds).  Under a mask the grid has two halves, like
// the KD row kernel's: workgroup i of the first half takes row i if the mask
// selects it and ends at once otherwise, so that the workgroups that read all
// start first; workgroup i of the second half zero-fills row i if the mask
// leaves it out.  No counting launch in front: a workgroup that computes
// counts the mask's few kilobytes itself while its loads are in flight.
// 4096 x 30522 bf16, us per call under a 15 % mask / without a mask (two sets
// of logits in turn, plain loads): 74 / 147 against 119 / - for the span kernel above;
// threads x vectors in flight 256 x 8: 77 / 157, 256 x 4: 80 / 165, 512 x 4:
// 77 / 147, 512 x 2: 78 / 152, 1024 x 4: 74 / 138 (but the zero-fill half alone
// 58 against 54), 1024 x 2: 78 / 140.
constexpr int kMseLongBlock = 512;
constexpr int kMseLongRegs = 8;     // 16-byte vectors per thread and operand in flight; half as many when the
                                    // gradient is a third operand (either way two workgroups fit a CU)
constexpr int64_t kMseLongMin = 8192;

template <typename T, bool ACC>
__global__ __launch_bounds__(kMseLongBlock) void mse_long_rows_kernel(const RowPieces tab,
                                                                      const uint8_t* __restrict__ mask,
                                                                      int64_t n_rows, int64_t V, float weight,
                                                                      int per_element, float* __restrict__ partial) {
  constexpr int accumulate = ACC ? 1 : 0;
  constexpr int REGS = ACC ? kMseLongRegs / 2 : kMseLongRegs;
  constexpr int VEC = 16 / sizeof(T);
  __shared__ float lds[kMseLongBlock / kWave];
  const int tid = threadIdx.x;
  int64_t row = blockIdx.x;
  const bool fill_half = row >= n_rows;
  if (fill_half) row -= n_rows;
  const bool sel = !mask || mask[row] != 0;
  if (fill_half == sel) return;  // uniform: the other half's row
  const RowPtrs<T> rp = row_ptrs<T>(tab, row);
  const T* sr = rp.a;
  const T* tr = rp.b;
  T* gr = rp.g;
  const T zero = from_f32<T>(0.f);
  if (!sel) {
    if (tid == 0) partial[row] = 0.f;
    if (!gr || accumulate) return;
    const uint32_t mis = (uint32_t)((uintptr_t)gr & 15u);
    int64_t head = (int64_t)(((16u - mis) & 15u) / sizeof(T));
    if (head > V) head = V;
    const int64_t nvec = (V - head) / VEC, tail0 = head + nvec * VEC;
    Vec16<T> z;
#pragma unroll
    for (int e = 0; e < VEC; ++e) z.v[e] = zero;
    if (tid < head) gr[tid] = zero;
    for (int64_t v = tid; v < nvec; v += kMseLongBlock) store16(gr + head + v * VEC, z);  // plain stores: a zero-fill
    if (tail0 + tid < V) gr[tail0 + tid] = zero;
    return;
  }

  const uint32_t mis = (uint32_t)((uintptr_t)sr & 15u);
  const bool alike = mis == (uint32_t)((uintptr_t)tr & 15u) && (!gr || mis == (uint32_t)((uintptr_t)gr & 15u)) &&
                     mis % sizeof(T) == 0;
  int64_t head = alike ? (int64_t)(((16u - mis) & 15u) / sizeof(T)) : V;
  if (head > V) head = V;
  const int64_t nvec = (V - head) / VEC, tail0 = head + nvec * VEC;
  const T* s4 = sr + head;
  const T* t4 = tr + head;
  T* g4 = gr + head;
  const bool acc_g = gr && accumulate;
  float acc = 0.f;
  float k = 0.f;
  for (int64_t base = 0; base < nvec || base == 0; base += (int64_t)kMseLongBlock * REGS) {
    Vec16<T> vs[REGS], vt[REGS], vg[ACC ? REGS : 1];
#pragma unroll
    for (int j = 0; j < REGS; ++j) {
      const int64_t v = base + tid + (int64_t)j * kMseLongBlock;
      if (v < nvec) {
        // read once: non-temporal loads (us per call, 15 % / 50 % / no mask: 73.6 / 112 / 146.5 -> 71 / 99.5 / 140.5)
        vs[j] = load16_stream(s4 + v * VEC);
        vt[j] = load16_stream(t4 + v * VEC);
        if (acc_g) vg[ACC ? j : 0] = load16(g4 + v * VEC);
      }
    }
    if (base == 0) {
      // the row count that scales the gradient, taken while the loads are in flight
      const float rows_sel = mask ? mask_count_block<kMseLongBlock>(mask, n_rows, lds) : (float)n_rows;
      k = 2.f * weight / (per_element ? rows_sel * (float)V : rows_sel);
      // the few elements in front of and behind the row's aligned middle (all of it when the operands
      // are aligned differently)
      for (int64_t i = tid; i < head; i += kMseLongBlock) {
        const T gv = mse_grad_one<T>(sr[i], tr[i], acc_g ? gr[i] : zero, k, accumulate, acc);
        if (gr) gr[i] = gv;
      }
      if (tail0 + tid < V) {
        const int64_t i = tail0 + tid;
        const T gv = mse_grad_one<T>(sr[i], tr[i], acc_g ? gr[i] : zero, k, accumulate, acc);
        if (gr) gr[i] = gv;
      }
    }
#pragma unroll
    for (int j = 0; j < REGS; ++j) {
      const int64_t v = base + tid + (int64_t)j * kMseLongBlock;
      if (v < nvec) {
        // one vector pair at a time out of registers the compiler can assume nothing about: otherwise it
        // unpacks every 16-bit vector to fp32 as it lands (176 registers, one workgroup per CU)
        u32x4 bs, bt;
        __builtin_memcpy(&bs, &vs[j], 16);
        __builtin_memcpy(&bt, &vt[j], 16);
        asm volatile("" : "+v"(bs), "+v"(bt));
        __builtin_memcpy(&vs[j], &bs, 16);
        __builtin_memcpy(&vt[j], &bt, 16);
        Vec16<T> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          o.v[e] = mse_grad_one<T>(vs[j].v[e], vt[j].v[e], acc_g ? vg[ACC ? j : 0].v[e] : zero, k, accumulate, acc);
        if (gr) {
          if (ACC)
            store16(g4 + v * VEC, o);
          else
            store16_stream(g4 + v * VEC, o);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const float tot = block_sum<kMseLongBlock / kWave>(acc, lds);
  if (tid == 0) partial[row] = tot;
}

inline int64_t mse_parts(int64_t V) { return (V + kMseSpan - 1) / kMseSpan; }

template <typename T>
int launch_mse(const RowPieces& tab, const uint8_t* mask, int64_t n_rows, int64_t V, float weight, int per_element,
               int accumulate, void* ws, float* loss_out, hipStream_t stream) {
  int* n_sel = reinterpret_cast<int*>(ws);
  float* partial = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + 16);
  if (V >= kMseLongMin && n_rows > 0) {
    const int64_t grid = mask ? 2 * n_rows : n_rows;
    if (grid * kMseLongBlock > 0xffffffffLL) return TS_ERR_RANGE;
    if (accumulate)
      hipLaunchKernelGGL((mse_long_rows_kernel<T, true>), dim3((unsigned)grid), dim3(kMseLongBlock), 0, stream, tab, mask,
                         n_rows, V, weight, per_element, partial);
    else
      hipLaunchKernelGGL((mse_long_rows_kernel<T, false>), dim3((unsigned)grid), dim3(kMseLongBlock), 0, stream, tab, mask,
                         n_rows, V, weight, per_element, partial);
    int rc = check_launch();
    if (rc) return rc;
    hipLaunchKernelGGL(mse_finalize_kernel, dim3(1), dim3(1024), 0, stream, partial, n_rows, (const int*)nullptr, mask,
                       n_rows, V, weight, per_element, accumulate, loss_out);
    return check_launch();
  }
  if (mask) {
    hipLaunchKernelGGL(mask_count_kernel, dim3(1), dim3(1024), 0, stream, mask, n_rows, n_sel);
    int rc = check_launch();
    if (rc) return rc;
  }
  // rows of up to 32 vectors (a ragged first and last one counted): 16 lanes each, else a wavefront
  const int64_t vecs = (V + Vec16<T>::N - 1) / Vec16<T>::N + 1;
  const int group = vecs <= 32 ? 16 : kWave;
  const int64_t per_block = kMseBlock / group;
  const int64_t blocks = (n_rows + per_block - 1) / per_block;
  if (blocks * kMseBlock > 0xffffffffLL) return TS_ERR_RANGE;
  const int* n_sel_arg = mask ? n_sel : (const int*)nullptr;
#define TS_MSE_LAUNCH(GROUP, ACC)                                                                              \
  hipLaunchKernelGGL((mse_rows_kernel<T, GROUP, ACC>), dim3((unsigned)blocks), dim3(kMseBlock), 0, stream, tab, \
                     mask, n_sel_arg, n_rows, V, weight, per_element, partial)
  if (group == 16) {
    if (accumulate) TS_MSE_LAUNCH(16, true); else TS_MSE_LAUNCH(16, false);
  } else {
    if (accumulate) TS_MSE_LAUNCH(kWave, true); else TS_MSE_LAUNCH(kWave, false);
  }
#undef TS_MSE_LAUNCH
  int rc = check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(mse_finalize_kernel, dim3(1), dim3(1024), 0, stream, partial, n_rows, n_sel_arg, mask, n_rows, V,
                     weight, per_element, accumulate, loss_out);
  return check_launch();
}

template <typename T>
int launch_cosine(const RowPieces& tab, const uint8_t* mask, int64_t n, int64_t c, float weight, void* ws,
                  float* loss_out, hipStream_t stream) {
  float* row_loss = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + 16);
  hipLaunchKernelGGL((cosine_rows_kernel<T>), dim3((unsigned)((n + 3) / 4)), dim3(256), 0, stream, tab, mask, n, c,
                     weight, row_loss);
  int rc = check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(cosine_finalize_kernel, dim3(1), dim3(1024), 0, stream, row_loss, n, weight, mask, loss_out);
  return check_launch();
}

template <typename T>
int launch_byol(const ByolArgs& args, int pairs, int64_t n, int64_t c, float* ws, float* loss_out,
                hipStream_t stream) {
  const int64_t total = pairs * n;
  const int64_t blocks = (total + 3) / 4;
  hipLaunchKernelGGL((byol_rows_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, args, pairs, n, c, ws);
  int rc = check_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(sum_scale_kernel, dim3(1), dim3(1024), 0, stream, ws, total, 1.0f,
                     (const int*)nullptr, (float)n, loss_out);
  return check_launch();
}

int byol_dispatch(const ByolArgs& args, int pairs, int64_t n, int64_t c, float* ws, float* loss_out, int dtype,
                  hipStream_t st) {
  switch (dtype) {
    case TS_F32: return launch_byol<float>(args, pairs, n, c, ws, loss_out, st);
    case TS_BF16: return launch_byol<bf16_t>(args, pairs, n, c, ws, loss_out, st);
    default: return launch_byol<f16_t>(args, pairs, n, c, ws, loss_out, st);
  }
}

inline size_t dtype_size(int dtype) { return dtype == TS_F32 ? 4 : 2; }

// out = scale * sum(v[0..n)) / denom on one workgroup (shared with infonce.hip)
int launch_sum_scale(const float* v, int64_t n, float scale, float denom, float* out, hipStream_t stream) {
  hipLaunchKernelGGL(sum_scale_kernel, dim3(1), dim3(1024), 0, stream, v, n, scale, (const int*)nullptr, denom,
                     out);
  return check_launch();
}

int cosine_dispatch(const RowPieces& tab, const uint8_t* mask, int64_t n, int64_t c, float weight, void* ws,
                    float* loss_out, int dtype, hipStream_t st) {
  if (n == 0) {
    hipLaunchKernelGGL(sum_scale_kernel, dim3(1), dim3(1024), 0, st, (const float*)ws, (int64_t)0, weight,
                       (const int*)nullptr, 0.f, loss_out);
    return check_launch();
  }
  switch (dtype) {
    case TS_F32: return launch_cosine<float>(tab, mask, n, c, weight, ws, loss_out, st);
    case TS_BF16: return launch_cosine<bf16_t>(tab, mask, n, c, weight, ws, loss_out, st);
    default: return launch_cosine<f16_t>(tab, mask, n, c, weight, ws, loss_out, st);
  }
}

int mse_dispatch(const RowPieces& tab, const uint8_t* mask, int64_t n_rows, int64_t V, float weight, int per_element,
                 int accumulate, void* ws, float* loss_out, int dtype, hipStream_t st) {
  if (n_rows == 0) {
    hipLaunchKernelGGL(mse_finalize_kernel, dim3(1), dim3(1024), 0, st, (const float*)ws, (int64_t)0,
                       (const int*)nullptr, (const uint8_t*)nullptr, (int64_t)0, V, weight, per_element, accumulate,
                       loss_out);
    return check_launch();
  }
  switch (dtype) {
    case TS_F32: return launch_mse<float>(tab, mask, n_rows, V, weight, per_element, accumulate, ws, loss_out, st);
    case TS_BF16: return launch_mse<bf16_t>(tab, mask, n_rows, V, weight, per_element, accumulate, ws, loss_out, st);
    default: return launch_mse<f16_t>(tab, mask, n_rows, V, weight, per_element, accumulate, ws, loss_out, st);
  }
}

}  // namespace ts

extern "C" {

size_t ts_cosine_workspace_bytes(int64_t n) {
  if (n < 0) n = 0;
  return (size_t)(16 + ((n * 4 + 15) / 16) * 16);
}

int ts_cosine_fwd_bwd(const void* x, const void* y, const uint8_t* row_mask, int64_t n, int64_t c, float weight,
                      void* workspace, float* loss_out, void* gx, int dtype, ts_stream_t stream) {
  // no rows, nothing to point at: the loss is then a mean over nothing, NaN
  if (!loss_out || (n > 0 && (!x || !y || !workspace))) return TS_ERR_ARG;
  if (n < 0 || c <= 0) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (n > (1 << 24)) return TS_ERR_RANGE;
  if ((uintptr_t)workspace & 15u) return TS_ERR_ALIGN;
  const ts::RowPieces tab = ts::row_single(x, y, gx, c, c, c);
  return ts::cosine_dispatch(tab, row_mask, n, c, weight, workspace, loss_out, dtype, (hipStream_t)stream);
}

int ts_cosine_pieces_fwd_bwd(const void* const* x_pieces, const void* const* y_pieces, void* const* gx_pieces,
                             const int64_t* piece_rows, int n_pieces, const uint8_t* row_mask, int64_t c, float weight,
                             void* workspace, float* loss_out, int dtype, ts_stream_t stream) {
  if (!workspace || !loss_out || c <= 0) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if ((uintptr_t)workspace & 15u) return TS_ERR_ALIGN;
  ts::RowPieces tab;
  int64_t n = 0;
  const int rc = ts::row_pieces(x_pieces, y_pieces, gx_pieces, piece_rows, n_pieces, c, ts::dtype_size(dtype), &tab, &n);
  if (rc) return rc;
  if (n > (1 << 24)) return TS_ERR_RANGE;
  return ts::cosine_dispatch(tab, row_mask, n, c, weight, workspace, loss_out, dtype, (hipStream_t)stream);
}

size_t ts_mse_workspace_bytes(int64_t n_rows, int64_t V) {
  if (n_rows < 0) n_rows = 0;
  if (V < 1) V = 1;
  return (size_t)(16 + ((n_rows * ts::mse_parts(V) * 4 + 15) / 16) * 16);
}

int ts_mse_fwd_bwd(const void* s, const void* t, const uint8_t* row_mask, int64_t n_rows, int64_t V, int64_t ld_s,
                   int64_t ld_t, float weight, int per_element, int accumulate, void* workspace, float* loss_out,
                   void* grad, int64_t ld_g, int dtype, ts_stream_t stream) {
  if (!loss_out || (n_rows > 0 && (!s || !t || !workspace))) return TS_ERR_ARG;
  if (n_rows < 0 || V <= 0 || ld_s < V || ld_t < V || (grad && ld_g < V)) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (n_rows > (1 << 24) || n_rows * ts::mse_parts(V) > 0x7fffffffLL) return TS_ERR_RANGE;
  if ((uintptr_t)workspace & 15u) return TS_ERR_ALIGN;
  const size_t es = ts::dtype_size(dtype);
  if (((uintptr_t)s | (uintptr_t)t | (uintptr_t)grad) & (es - 1)) return TS_ERR_ALIGN;
  const ts::RowPieces tab = ts::row_single(s, t, grad, ld_s, ld_t, ld_g);
  return ts::mse_dispatch(tab, row_mask, n_rows, V, weight, per_element, accumulate, workspace, loss_out, dtype,
                          (hipStream_t)stream);
}

int ts_mse_pieces_fwd_bwd(const void* const* s_pieces, const void* const* t_pieces, void* const* grad_pieces,
                          const int64_t* piece_rows, int n_pieces, const uint8_t* row_mask, int64_t V, float weight,
                          int per_element, int accumulate, void* workspace, float* loss_out, int dtype,
                          ts_stream_t stream) {
  if (!workspace || !loss_out || V <= 0) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if ((uintptr_t)workspace & 15u) return TS_ERR_ALIGN;
  ts::RowPieces tab;
  int64_t n_rows = 0;
  const int rc = ts::row_pieces(s_pieces, t_pieces, grad_pieces, piece_rows, n_pieces, V, ts::dtype_size(dtype), &tab,
                                &n_rows);
  if (rc) return rc;
  if (n_rows > (1 << 24) || n_rows * ts::mse_parts(V) > 0x7fffffffLL) return TS_ERR_RANGE;
  return ts::mse_dispatch(tab, row_mask, n_rows, V, weight, per_element, accumulate, workspace, loss_out, dtype,
                          (hipStream_t)stream);
}


int ts_scale_rows(void* grad, int64_t n_rows, int64_t V, int64_t ld_g, const float* g_dev, int dtype,
                  ts_stream_t stream) {
  if (!g_dev || n_rows < 0 || V < 0 || ld_g < V) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  if (n_rows == 0 || V == 0) return TS_OK;
  if (!grad) return TS_ERR_ARG;
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
  if (!loss_out || (n > 0 && (!x1 || !y1 || !workspace))) return TS_ERR_ARG;
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
  ts::ByolArgs args = {};
  args.n_pieces = 1;
  args.x[0][0] = x1;
  args.y[0][0] = y1;
  args.g[0][0] = gx1;
  args.x[1][0] = x2;
  args.y[1][0] = y2;
  args.g[1][0] = gx2;
  return ts::byol_dispatch(args, x2 ? 2 : 1, n, c, workspace, loss_out, dtype, st);
}

int ts_byol_pieces_fwd_bwd(const void* const* x1_pieces, const void* const* y1_pieces, void* const* gx1_pieces,
                           const void* const* x2_pieces, const void* const* y2_pieces, void* const* gx2_pieces,
                           const int64_t* piece_rows, int n_pieces, int64_t c, float* workspace, float* loss_out,
                           int dtype, ts_stream_t stream) {
  if (!x1_pieces || !y1_pieces || !piece_rows || !workspace || !loss_out) return TS_ERR_ARG;
  if ((x2_pieces == nullptr) != (y2_pieces == nullptr)) return TS_ERR_ARG;
  if (n_pieces < 1 || n_pieces > ts::kByolMaxPieces) return TS_ERR_RANGE;
  if (c <= 0) return TS_ERR_ARG;
  if (dtype != TS_F32 && dtype != TS_BF16 && dtype != TS_F16) return TS_ERR_ARG;
  const int pairs = x2_pieces ? 2 : 1;
  ts::ByolArgs args = {};
  args.n_pieces = n_pieces;
  int64_t n = 0;
  for (int p = 0; p < pairs; ++p) {
    const void* const* xs = p ? x2_pieces : x1_pieces;
    const void* const* ys = p ? y2_pieces : y1_pieces;
    void* const* gs = p ? gx2_pieces : gx1_pieces;
    const bool want = gs && gs[0];
    int64_t rows = 0;
    for (int i = 0; i < n_pieces; ++i) {
      if (piece_rows[i] <= 0 || !xs[i] || !ys[i]) return TS_ERR_ARG;
      if (want != (gs && gs[i] != nullptr)) return TS_ERR_ARG;
      args.row0[i] = rows;
      args.x[p][i] = xs[i];
      args.y[p][i] = ys[i];
      args.g[p][i] = want ? gs[i] : nullptr;
      rows += piece_rows[i];
    }
    n = rows;
  }
  if (n > (1 << 28)) return TS_ERR_RANGE;
  return ts::byol_dispatch(args, pairs, n, c, workspace, loss_out, dtype, (hipStream_t)stream);
}

}  // extern "C"
