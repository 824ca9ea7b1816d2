// A consumer of the C ABI that knows nothing of Python or PyTorch: plain HIP
// runtime calls for memory, include/tspipe_amd.h for everything else.  Checks
// the EMA bit for bit against one-rounding-per-operation host arithmetic and
// the KD soft-target loss against a double-precision evaluation, gathers a few
// small pieces without a table, asks for a loss over zero rows, then prints
// "c-abi consumer: ok".  Built by __graft_entry__.build(), run by the GPU tests.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/tspipe_amd.h"

#define HIP_OK(call)                                                              \
  do {                                                                            \
    hipError_t e_ = (call);                                                       \
    if (e_ != hipSuccess) {                                                       \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));      \
      std::exit(2);                                                               \
    }                                                                             \
  } while (0)
#define TS_OK_(call)                                                              \
  do {                                                                            \
    int s_ = (int)(call);                                                         \
    if (s_ < 0) {                                                                 \
      std::fprintf(stderr, "%s -> %d (%s)\n", #call, s_, ts_error_string(s_));    \
      std::exit(3);                                                               \
    }                                                                             \
  } while (0)

static uint32_t rng_state = 12345u;
static float frand() {  // uniform in [-1, 1)
  rng_state = rng_state * 1664525u + 1013904223u;
  return (float)((rng_state >> 8) & 0xffffff) / 8388608.0f - 1.0f;
}

static int check_ema(hipStream_t stream) {
  // three "parameters" of awkward sizes, one empty
  const int64_t numels[4] = {1000003, 0, 77, 4096};
  const int n = 4;
  const float m32 = (float)0.996, c32 = (float)(1.0 - 0.996);
  std::vector<std::vector<float>> t(n), s(n);
  const void* tp[4];
  const void* sp[4];
  void* op[4];
  for (int i = 0; i < n; ++i) {
    t[i].resize(numels[i]);
    s[i].resize(numels[i]);
    for (auto& v : t[i]) v = frand() * 0.02f;
    for (auto& v : s[i]) v = frand() * 0.02f;
    void *dt = nullptr, *ds = nullptr, *dout = nullptr;
    const size_t bytes = (size_t)numels[i] * 4 + 16;
    HIP_OK(hipMalloc(&dt, bytes));
    HIP_OK(hipMalloc(&ds, bytes));
    HIP_OK(hipMalloc(&dout, bytes));
    HIP_OK(hipMemcpy(dt, t[i].data(), (size_t)numels[i] * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(ds, s[i].data(), (size_t)numels[i] * 4, hipMemcpyHostToDevice));
    tp[i] = dt;
    sp[i] = ds;
    op[i] = dout;
  }
  int64_t total = 0;
  for (int i = 0; i < n; ++i) total += numels[i];
  const int64_t chunk = ts_ema_auto_chunk(total);
  const int64_t count = ts_ema_plan(tp, sp, op, numels, n, chunk, nullptr, 0);
  TS_OK_(count);
  ts_ema_chunk* host_table = nullptr;
  HIP_OK(hipHostMalloc((void**)&host_table, (size_t)count * sizeof(ts_ema_chunk), hipHostMallocDefault));
  TS_OK_(ts_ema_plan(tp, sp, op, numels, n, chunk, host_table, count));
  ts_ema_chunk* dev_table = nullptr;
  HIP_OK(hipMalloc((void**)&dev_table, (size_t)count * sizeof(ts_ema_chunk)));
  HIP_OK(hipMemcpyAsync(dev_table, host_table, (size_t)count * sizeof(ts_ema_chunk), hipMemcpyHostToDevice, stream));
  TS_OK_(ts_ema_multi(dev_table, count, chunk, m32, c32, stream));
  HIP_OK(hipStreamSynchronize(stream));
  int bad = 0;
  for (int i = 0; i < n; ++i) {
    std::vector<float> got(numels[i]);
    HIP_OK(hipMemcpy(got.data(), op[i], (size_t)numels[i] * 4, hipMemcpyDeviceToHost));
    for (int64_t j = 0; j < numels[i]; ++j) {
      volatile float a = t[i][j] * m32;  // one rounding per operation, no contraction
      volatile float b = s[i][j] * c32;
      const float want = a + b;
      if (std::memcmp(&want, &got[j], 4) != 0 && ++bad < 5)
        std::fprintf(stderr, "ema mismatch tensor %d elem %lld: %a vs %a\n", i, (long long)j, got[j], want);
    }
  }
  return bad;
}

static int check_kd(hipStream_t stream) {
  const int64_t rows = 256, V = 100;
  const float T = 4.0f;
  std::vector<float> s(rows * V), t(rows * V);
  for (auto& v : s) v = frand() * 3.f;
  for (auto& v : t) v = frand() * 3.f;
  void *ds, *dt, *dg, *ws;
  float* dloss;
  HIP_OK(hipMalloc(&ds, s.size() * 4));
  HIP_OK(hipMalloc(&dt, t.size() * 4));
  HIP_OK(hipMalloc(&dg, s.size() * 4));
  HIP_OK(hipMalloc(&ws, ts_kd_workspace_bytes(rows, V, TS_F32)));
  HIP_OK(hipMalloc((void**)&dloss, 4));
  HIP_OK(hipMemcpy(ds, s.data(), s.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dt, t.data(), t.size() * 4, hipMemcpyHostToDevice));
  TS_OK_(ts_kd_fwd_bwd(ds, dt, nullptr, rows, V, V, V, 1.0f / T, T * T, ws, dloss, dg, V, TS_F32, stream));
  HIP_OK(hipStreamSynchronize(stream));
  float loss;
  std::vector<float> g(s.size());
  HIP_OK(hipMemcpy(&loss, dloss, 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(g.data(), dg, g.size() * 4, hipMemcpyDeviceToHost));
  // double-precision evaluation of T^2 * KL(softmax(t/T) || softmax(s/T)), batch mean
  double want = 0.0, gmax = 0.0, gerr = 0.0;
  for (int64_t r = 0; r < rows; ++r) {
    double ms = -1e300, mt = -1e300, zs = 0, zt = 0;
    for (int64_t v = 0; v < V; ++v) {
      ms = std::fmax(ms, s[r * V + v] / (double)T);
      mt = std::fmax(mt, t[r * V + v] / (double)T);
    }
    for (int64_t v = 0; v < V; ++v) {
      zs += std::exp(s[r * V + v] / (double)T - ms);
      zt += std::exp(t[r * V + v] / (double)T - mt);
    }
    for (int64_t v = 0; v < V; ++v) {
      const double ls = s[r * V + v] / (double)T - ms - std::log(zs);
      const double lt = t[r * V + v] / (double)T - mt - std::log(zt);
      const double p = std::exp(lt), q = std::exp(ls);
      want += p * (lt - ls);
      const double gw = (double)T * (q - p) / (double)rows;  // T^2 * (q - p) / T / rows
      gmax = std::fmax(gmax, std::fabs(gw));
      gerr = std::fmax(gerr, std::fabs(gw - (double)g[r * V + v]));
    }
  }
  want = want * T * T / rows;
  int bad = 0;
  if (std::fabs(loss - want) > 1e-5 * std::fabs(want)) {
    std::fprintf(stderr, "kd loss %.9g vs %.9g\n", loss, want);
    ++bad;
  }
  if (gerr > 1e-5 * gmax) {
    std::fprintf(stderr, "kd gradient error %.3g (peak %.3g)\n", gerr, gmax);
    ++bad;
  }
  return bad;
}

// A gather of a few small pieces without a table: odd byte counts, an empty segment, unaligned starts.
static int check_copy_few(hipStream_t stream) {
  const int64_t bytes[4] = {4099, 0, 65536, 7};
  const int64_t src_off[4] = {0, 0, 3, 1}, total = 4099 + 65536 + 7;
  std::vector<std::vector<unsigned char>> host(4);
  const void* src[4];
  void* dst[4];
  unsigned char* joined = nullptr;
  HIP_OK(hipMalloc((void**)&joined, (size_t)total + 16));
  HIP_OK(hipMemset(joined, 0xee, (size_t)total + 16));
  int64_t at = 0;
  for (int i = 0; i < 4; ++i) {
    host[i].resize((size_t)bytes[i]);
    for (auto& v : host[i]) v = (unsigned char)(frand() * 127.f + 128.f);
    unsigned char* d = nullptr;
    HIP_OK(hipMalloc((void**)&d, (size_t)bytes[i] + 32));
    if (bytes[i]) HIP_OK(hipMemcpy(d + src_off[i], host[i].data(), (size_t)bytes[i], hipMemcpyHostToDevice));
    src[i] = d + src_off[i];
    dst[i] = joined + at;
    at += bytes[i];
  }
  TS_OK_(ts_copy_few(src, dst, bytes, 4, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<unsigned char> got((size_t)total + 16);
  HIP_OK(hipMemcpy(got.data(), joined, got.size(), hipMemcpyDeviceToHost));
  int bad = 0;
  at = 0;
  for (int i = 0; i < 4; ++i) {
    if (bytes[i] && std::memcmp(got.data() + at, host[i].data(), (size_t)bytes[i]) != 0) {
      std::fprintf(stderr, "copy_few: segment %d differs\n", i);
      ++bad;
    }
    at += bytes[i];
  }
  for (int64_t j = total; j < total + 16; ++j)
    if (got[(size_t)j] != 0xee) {
      std::fprintf(stderr, "copy_few: wrote past the end at %lld\n", (long long)j);
      ++bad;
      break;
    }
  if (ts_copy_few(src, dst, bytes, 17, stream) != TS_ERR_RANGE) ++bad;
  return bad;
}

// A loss over zero rows is a mean over nothing: NaN, no error, input pointers not needed.
static int check_kd_zero_rows(hipStream_t stream) {
  void* ws;
  float* dloss;
  HIP_OK(hipMalloc(&ws, ts_kd_workspace_bytes(0, 100, TS_F32)));
  HIP_OK(hipMalloc((void**)&dloss, 4));
  HIP_OK(hipMemset(dloss, 0, 4));
  TS_OK_(ts_kd_fwd_bwd(nullptr, nullptr, nullptr, 0, 100, 100, 100, 0.25f, 16.f, ws, dloss, nullptr, 100, TS_F32, stream));
  HIP_OK(hipStreamSynchronize(stream));
  float loss = 0.f;
  HIP_OK(hipMemcpy(&loss, dloss, 4, hipMemcpyDeviceToHost));
  if (!std::isnan(loss)) {
    std::fprintf(stderr, "kd over zero rows gave %g, not NaN\n", loss);
    return 1;
  }
  return 0;
}

int main() {
  std::printf("%s\n", ts_version());
  HIP_OK(hipSetDevice(0));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  const int bad = check_ema(stream) + check_kd(stream) + check_copy_few(stream) + check_kd_zero_rows(stream);
  // error paths answer with a status, not a crash
  if (ts_ema_multi(nullptr, 1, 1024, 0.5f, 0.5f, stream) != TS_ERR_ARG) return 4;
  if (ts_ema_multi(nullptr, 0, 1000, 0.5f, 0.5f, stream) != TS_ERR_ARG) return 5;  // chunk not a multiple of 1024
  if (bad) {
    std::printf("c-abi consumer: %d mismatches\n", bad);
    return 1;
  }
  std::printf("c-abi consumer: ok\n");
  return 0;
}
