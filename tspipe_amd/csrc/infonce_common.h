// Declarations shared by the two InfoNCE implementations: the bf16-MFMA path
// (infonce.hip) and the fp32-MFMA path for fp32 inputs, other widths and small
// temperatures (infonce_general.hip).
#pragma once

#include "common.h"

namespace ts {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr float kNceLog2e = 1.4426950408889634f;
constexpr float kNceLn2 = 0.6931471805599453f;
constexpr float kNormEps = 1e-12f;  // F.normalize's eps
constexpr int kNceMaxPieces = 8;

__host__ __device__ inline int64_t nce_round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
inline size_t nce_align(size_t x) { return (x + 255) & ~(size_t)255; }

// One (q, k) pair's pointers; the kernels pick theirs by blockIdx.z, so the two
// pairs of the symmetric loss share every launch.  q, k and dq may come as up
// to kNceMaxPieces row blocks (micro-batch outputs that were never
// concatenated): piece i holds rows row0[i] .. row0[i+1]-1.  n_pieces == 0
// means the single matrices q / k / dq.
struct NcePair {
  const void* q;
  const void* k;
  void* dq;
  float *rq, *rk, *pdiag, *lpart, *opart;
  uint16_t* khat;  // normalised keys, bf16, [npad][C]            (bf16 path)
  uint16_t* qb;    // bf16 copy of the queries for fp16 inputs, else null  (bf16 path)
  float* stat;     // per key split and row: running maximum, sum over the negatives, positive term, positive logit (fp32 path)
  int n_pieces;
  int64_t row0[kNceMaxPieces];
  const void* qp[kNceMaxPieces];
  const void* kp[kNceMaxPieces];
  void* dqp[kNceMaxPieces];
};
struct NceArgs {
  NcePair p[2];
};

struct NceRow {
  const void* q;
  const void* k;
  void* dq;
};

// Pointers to one batch row of q, k and dq (T: the storage type).
template <typename T>
__device__ __forceinline__ NceRow nce_row(const NcePair& pr, int64_t row, int C) {
  NceRow r;
  if (pr.n_pieces == 0) {
    r.q = (const T*)pr.q + row * C;
    r.k = (const T*)pr.k + row * C;
    r.dq = pr.dq ? (T*)pr.dq + row * C : nullptr;
    return r;
  }
  const void* qb = pr.qp[0];
  const void* kb = pr.kp[0];
  void* db = pr.dqp[0];
  int64_t r0 = 0;
#pragma unroll
  for (int i = 1; i < kNceMaxPieces; ++i) {
    const bool ge = i < pr.n_pieces && row >= pr.row0[i];
    qb = ge ? pr.qp[i] : qb;
    kb = ge ? pr.kp[i] : kb;
    db = ge ? pr.dqp[i] : db;
    r0 = ge ? pr.row0[i] : r0;
  }
  const int64_t local = row - r0;
  r.q = (const T*)qb + local * C;
  r.k = (const T*)kb + local * C;
  r.dq = db ? (T*)db + local * C : nullptr;
  return r;
}

// The fp32-MFMA path (infonce_general.hip): any width up to 512, any
// temperature, products and sums in fp32.  args holds q / k / dq (or their
// pieces); the workspace pointers are filled in by the launcher.
// Workgroups the main kernels aim to put on the chip (ts_infonce_set_workgroup_target):
// the number of key splits follows from it.  kNceMaxWorkgroupTarget, one per
// CU, is the default and what the workspace is sized for.
constexpr int kNceMaxWorkgroupTarget = 256;
int nce_workgroup_target();

size_t nce_general_workspace_bytes(int64_t n, int64_t c, int n_pairs);
int nce_general_launch(NceArgs& args, int pairs, int64_t n, int64_t c, float tau, void* workspace, float* loss_out,
                       int dtype, hipStream_t stream);

}  // namespace ts
