// C++ correctness-and-benchmark harness for libfmha_i8.so.  Plays the role of the reference's test driver
// (test_fmha_i8.cpp:19-312: generate data, CPU path, H2D, warm-up, timed call, compare) with what that driver lacks:
// a run-time CLI, an int8 CPU checker with an LSB histogram, many timed iterations, the CPU path timed with its
// core count, and one JSON record per case.  Host code only: it calls the library through include/fmha_i8.h exactly
// as the reference's driver calls gpuImpl::FMHAInferI8 (test_fmha_i8.cpp:204-222).
//
//   test_fmha_i8 --config 3                 one of the five benchmark configurations
//   test_fmha_i8 --sweep                    the reference's own sweep: B=H=1, S in {64,128,...,512,1024,2048,4096}, d in {64,128},
//                                           uniform(+-0.5) Q/K, |uniform| V, scattered 20 % mask, o_amax measured
//   test_fmha_i8 --B 2 --H 4 --S 512 --d 64 [--valid L | --pad none|bert|tail16th|scatter] [--dist normal|student_t|reference]
//   ... --Sq 100                            that many query rows per head over the S keys (FMHAInferI8Cross)
//   ... --full-range-p                      P on 255 steps (FMHAInferI8CrossFullRangeP), checked against that mode of the checker
//   common: --seed N --iters N --warmup N --cpu-heads N (0 = all) --cpu-threads N --json FILE --no-check
//   --quant MiB            instead of attention cases: abs-max, quantise and de-quantise (include/fmha_quant.h) over that
//                          many MiB of fp32 input, checked bit for bit against the CPU checker and timed against HBM
//   --calibrate-copy MiB   also run one device-to-device copy of that size, so that a counter run (FETCH_SIZE /
//                          WRITE_SIZE) sees a plain copy kernel of known traffic to scale the attention kernel's by
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include <unistd.h>

#include "fmha_i8.h"
#include "fmha_quant.h"
#include "fmha_oracle.hpp"

inline void check_hip(hipError_t e, const char* file, int line) {
  if (e != hipSuccess) {
    fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e), file, line);
    exit(3);
  }
}
#define CHECK_HIP(x) check_hip((x), __FILE__, __LINE__)

namespace {

constexpr double kInt8PeakTops = 5033.2;  // 256 CU x 8192 op/clk/CU x 2.4 GHz

struct Rng {  // splitmix64 -> uniform -> Box-Muller; identical on every machine, unlike <random> distributions
  uint64_t s;
  explicit Rng(uint64_t seed) : s(seed) {}
  uint64_t next() {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
  double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
  double normal() {
    double u1 = uniform(), u2 = uniform();
    if (u1 < 1e-300) u1 = 1e-300;
    return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
  }
  double student_t3() {
    const double z = normal(), a = normal(), b = normal(), c = normal();
    return z / std::sqrt((a * a + b * b + c * c) / 3.0);
  }
};

struct Case {
  std::string name;
  int B = 1, H = 1, S = 128, d = 64;
  int Sq = 0;                   // query rows per head when they differ from S (0: self-attention, the reference's case)
  std::string dist = "normal";  // normal | student_t | reference
  double sigma = 1.0;
  std::string pad = "none";     // none | bert | tail16th | scatter | valid
  int valid = -1;
  bool measured_o_amax = false;
};

Case config_case(int id) {
  Case c;
  c.name = "C" + std::to_string(id);
  switch (id) {
    case 1: c.B = 1, c.H = 2, c.S = 128, c.d = 64; break;
    case 2: c.B = 8, c.H = 12, c.S = 512, c.d = 64, c.pad = "bert"; break;
    case 3: c.B = 4, c.H = 16, c.S = 1024, c.d = 128; break;
    case 4: c.B = 1, c.H = 32, c.S = 4096, c.d = 128, c.sigma = 0.5, c.pad = "tail16th"; break;
    case 5: c.B = 16, c.H = 16, c.S = 2048, c.d = 64, c.dist = "student_t", c.sigma = 0.5; break;
    default: fprintf(stderr, "--config takes 1..5\n"); exit(2);
  }
  return c;
}

struct Options {
  uint64_t seed = 2023;  // test_fmha_i8.cpp:49
  int iters = 1000;
  int warmup = 1500;
  long cpu_heads = 8;
  int cpu_threads = 0;
  bool check = true;
  bool full_range_p = false;
  std::string json;
};

struct Data {
  std::vector<float> qf, kf, vf;
  std::vector<int8_t> q, k, v, mask;
  float q_amax, k_amax, v_amax;
};

Data generate(const Case& c, uint64_t seed) {
  Data t;
  const long n = (long)c.B * c.H * c.S * c.d, nq = (long)c.B * c.H * (c.Sq > 0 ? c.Sq : c.S) * c.d;
  t.qf.resize(nq), t.kf.resize(n), t.vf.resize(n);
  t.q.resize(nq), t.k.resize(n), t.v.resize(n);
  t.mask.assign((long)c.B * c.S, 0);
  Rng rm(seed * 1000003ull + 4), rq(seed * 1000003ull + 1), rk(seed * 1000003ull + 2), rv(seed * 1000003ull + 3);
  for (int b = 0; b < c.B; ++b) {
    int L = c.S;
    if (c.pad == "bert") L = 64 * (int)(c.S / 128 + rm.next() % (c.S / 128 + 1));  // [S/2, S], multiple of 64
    if (c.pad == "tail16th") L = c.S - c.S / 16;
    if (c.pad == "valid") L = c.valid;
    for (int j = 0; j < c.S; ++j)
      t.mask[(long)b * c.S + j] = c.pad == "scatter" ? (rm.uniform() < 0.2 ? 1 : 0) : (j >= L ? 1 : 0);
  }
  for (long i = 0; i < nq; ++i) {
    if (c.dist == "reference") t.qf[i] = (float)(rq.uniform() - 0.5);  // test_fmha_i8.cpp:81-89
    else if (c.dist == "student_t") t.qf[i] = (float)(c.sigma * rq.student_t3());
    else t.qf[i] = (float)(c.sigma * rq.normal());
  }
  for (long i = 0; i < n; ++i) {
    if (c.dist == "reference") {
      t.kf[i] = (float)(rk.uniform() - 0.5);
      t.vf[i] = (float)std::fabs(rv.uniform() - 0.5);
    } else if (c.dist == "student_t") {
      t.kf[i] = (float)(c.sigma * rk.student_t3());
      t.vf[i] = (float)rv.normal();
    } else {
      t.kf[i] = (float)(c.sigma * rk.normal());
      t.vf[i] = (float)(c.sigma * rv.normal());
    }
  }
  t.q_amax = fmha_oracle::abs_max(t.qf.data(), nq);  // test_fmha_i8.cpp:95-110
  t.k_amax = fmha_oracle::abs_max(t.kf.data(), n);
  t.v_amax = fmha_oracle::abs_max(t.vf.data(), n);
  for (long i = 0; i < nq; ++i) t.q[i] = (int8_t)fmha_oracle::quantize_i8(t.qf[i], t.q_amax);
  for (long i = 0; i < n; ++i) {
    t.k[i] = (int8_t)fmha_oracle::quantize_i8(t.kf[i], t.k_amax);
    t.v[i] = (int8_t)fmha_oracle::quantize_i8(t.vf[i], t.v_amax);
  }
  return t;
}

double seconds_since(std::chrono::steady_clock::time_point t0) {
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

bool run_case(const Case& c, const Options& opt, FILE* json) {
  const bool full = opt.full_range_p;
  const bool cross = full || (c.Sq > 0 && c.Sq != c.S);  // queries and keys differ in number: FMHAInferI8Cross
  const int Sq = c.Sq > 0 ? c.Sq : c.S;
  const bool square = Sq == c.S;  // the reference's float path and its acceptance metric apply
  printf("compute type=int32, data type=int8, batch_num=%d, seq_len=%d, head_num=%d, head_dim=%d, dist=%s, pad=%s",
         c.B, c.S, c.H, c.d, c.dist.c_str(), c.pad.c_str());
  if (cross) printf(", query rows=%d", Sq);
  if (full) printf(", P on 255 steps");
  printf("\n");
  fflush(stdout);
  Data t = generate(c, opt.seed);
  const long n = (long)c.B * c.H * c.S * c.d, nq = (long)c.B * c.H * Sq * c.d, heads = (long)c.B * c.H;
  const long cpu_heads = (opt.cpu_heads <= 0 || opt.cpu_heads > heads) ? heads : opt.cpu_heads;
  const int threads = opt.cpu_threads > 0 ? opt.cpu_threads : (int)std::thread::hardware_concurrency();

  // ---- CPU float path of the reference driver (test_fmha_i8.cpp:141-162), timed, on the sampled heads ------------
  std::vector<float> o_ref(nq, 0.f);
  float o_amax = 1.0f;
  double cpu_fp32_s = 0, cpu_i8_s = 0;
  if (opt.check && square) {  // (the reference's float path is square: S queries over S keys)
    auto t0 = std::chrono::steady_clock::now();
    fmha_oracle::fmha_fp32_cpu(t.qf.data(), t.kf.data(), t.vf.data(), t.mask.data(), o_ref.data(), c.B, c.H, c.S, c.d,
                               threads, 0, cpu_heads);
    cpu_fp32_s = seconds_since(t0);
    if (c.measured_o_amax) o_amax = fmha_oracle::abs_max(o_ref.data(), cpu_heads * c.S * c.d);  // :161
  }

  // ---- device buffers, H2D (test_fmha_i8.cpp:165-178) ------------------------------------------------------------
  void *dq, *dk, *dv, *dm, *dout;
  CHECK_HIP(hipMalloc(&dq, nq)), CHECK_HIP(hipMalloc(&dk, n)), CHECK_HIP(hipMalloc(&dv, n));
  CHECK_HIP(hipMalloc(&dout, nq)), CHECK_HIP(hipMalloc(&dm, (size_t)c.B * c.S));
  CHECK_HIP(hipMemcpy(dq, t.q.data(), nq, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dk, t.k.data(), n, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dv, t.v.data(), n, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dm, t.mask.data(), (size_t)c.B * c.S, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemset(dout, 0, nq));
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));

  FMHAParamI8 param;  // test_fmha_i8.cpp:180-192
  param.q_amax = t.q_amax, param.k_amax = t.k_amax, param.v_amax = t.v_amax, param.o_amax = o_amax;
  AttnDataDescriptor desc;
  desc.batch_num = c.B, desc.seq_len = c.S, desc.head_num = c.H, desc.head_dim = c.d;
  printf("q_amax: %g  k_amax: %g  v_amax: %g  o_amax: %g\n", t.q_amax, t.k_amax, t.v_amax, o_amax);

  FMHACrossAttnDescriptor xdesc;
  xdesc.batch_num = c.B, xdesc.seq_len_q = Sq, xdesc.seq_len_kv = c.S, xdesc.head_num = c.H, xdesc.head_dim = c.d;
  auto call = [&]() {
    if (full) (void)FMHAInferI8CrossFullRangeP(stream, param, xdesc, dq, dk, dv, dm, dout);
    else if (cross) (void)FMHAInferI8Cross(stream, param, xdesc, dq, dk, dv, dm, dout);
    else gpuImpl::FMHAInferI8(stream, param, desc, dq, dk, dv, dm, dout, true);
  };
  const int st = full    ? FMHAInferI8CrossFullRangeP(stream, param, xdesc, dq, dk, dv, dm, dout)
                 : cross ? FMHAInferI8Cross(stream, param, xdesc, dq, dk, dv, dm, dout)
                         : FMHAInferI8Status(stream, param, desc, dq, dk, dv, dm, dout, true);  // warm-up, checked
  if (st != FMHA_I8_OK) {
    fprintf(stderr, "launch failed: %s\n", FMHAInferI8StatusString(st));
    return false;
  }
  // warm-up: the shader clock needs tens of milliseconds of load to settle (a cold call is up to 30 % slower)
  for (int i = 0; i < opt.warmup; ++i) call();
  CHECK_HIP(hipStreamSynchronize(stream));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0)), CHECK_HIP(hipEventCreate(&e1));
  CHECK_HIP(hipEventRecord(e0, stream));
  for (int i = 0; i < opt.iters; ++i) call();
  CHECK_HIP(hipEventRecord(e1, stream));
  CHECK_HIP(hipEventSynchronize(e1));
  float ms_total = 0;
  CHECK_HIP(hipEventElapsedTime(&ms_total, e0, e1));
  const double us_mean = ms_total * 1e3 / opt.iters;
  std::vector<float> singles;
  for (int i = 0; i < 20; ++i) {
    CHECK_HIP(hipEventRecord(e0, stream));
    call();
    CHECK_HIP(hipEventRecord(e1, stream));
    CHECK_HIP(hipEventSynchronize(e1));
    float ms1;
    CHECK_HIP(hipEventElapsedTime(&ms1, e0, e1));
    singles.push_back(ms1 * 1e3f);
  }
  std::sort(singles.begin(), singles.end());
  const double ops = 4.0 * c.B * c.H * (double)Sq * c.S * c.d;
  const double tops = ops / us_mean * 1e-6;
  printf("FMHA Inference took %.3f us/call (mean of %d), single-call min %.3f median %.3f us, %.1f TOPS, %.2f %% of "
         "%.1f TOPS int8 peak, %.1f GB/s\n",
         us_mean, opt.iters, singles.front(), singles[singles.size() / 2], tops, 100 * tops / kInt8PeakTops,
         kInt8PeakTops, (2.0 * n + 2.0 * nq) / us_mean * 1e-3);

  std::vector<int8_t> o(nq);
  CHECK_HIP(hipMemcpy(o.data(), dout, nq, hipMemcpyDeviceToHost));
  CHECK_HIP(hipFree(dq)), CHECK_HIP(hipFree(dk)), CHECK_HIP(hipFree(dv)), CHECK_HIP(hipFree(dm));
  CHECK_HIP(hipFree(dout));
  CHECK_HIP(hipEventDestroy(e0)), CHECK_HIP(hipEventDestroy(e1)), CHECK_HIP(hipStreamDestroy(stream));

  bool pass = true;
  long hist[4] = {0, 0, 0, 0};
  float dev_pct = 0;
  if (opt.check) {
    std::vector<int8_t> want(nq, 0);
    auto t0 = std::chrono::steady_clock::now();
    fmha_oracle::fmha_i8_cpu_blockwise_cross(t.q.data(), t.k.data(), t.v.data(), t.mask.data(), want.data(), c.B, c.H,
                                             Sq, c.S, c.d, t.q_amax, t.k_amax, t.v_amax, o_amax,
                                             (c.S + 63) / 64 * 64 % 128 == 0 ? 128 : 64, threads, 0, cpu_heads, full);
    cpu_i8_s = seconds_since(t0);
    const long m = cpu_heads * Sq * c.d;
    int worst = 0;
    for (long i = 0; i < m; ++i) {
      const int dl = std::abs((int)o[i] - (int)want[i]);
      hist[std::min(dl, 3)]++;
      worst = std::max(worst, dl);
    }
    const double within1 = (double)(hist[0] + hist[1]) / m;
    if (square) dev_pct = fmha_oracle::mean_rel_deviation_pct(o.data(), o_ref.data(), m, o_amax);  // inc/utils.hpp:59-89
    pass = within1 >= 0.999 && worst <= 2 && (!square || !c.measured_o_amax || dev_pct < 20.f);
    printf("parity vs int8 CPU checker on %ld of %ld heads: delta 0: %ld, 1: %ld, 2: %ld, >2: %ld -> within 1 LSB "
           "%.5f, max %d  [%s]\n", cpu_heads, heads, hist[0], hist[1], hist[2], hist[3], within1, worst,
           pass ? "PASS" : "FAIL");
    if (square)
      printf("INT8 average absolute deviation vs float path: %f %%%s\n", dev_pct,
             c.measured_o_amax ? " (reference criterion: < 20)" : " (o_amax fixed at 1: reported only)");
    printf("CPU: float path %.3f s, int8 checker %.3f s, %ld heads, %d threads\n", cpu_fp32_s, cpu_i8_s, cpu_heads,
           threads);
  }
  if (json)
    fprintf(json,
            "{\"case\":\"%s\",\"B\":%d,\"H\":%d,\"S\":%d,\"Sq\":%d,\"d\":%d,\"dist\":\"%s\",\"pad\":\"%s\",\"seed\":%llu,"
            "\"mask_polarity\":\"reference (nonzero = masked out)\",\"us_per_call\":%.4f,\"us_single_min\":%.4f,"
            "\"us_single_median\":%.4f,\"tops\":%.3f,\"pct_of_int8_peak\":%.3f,\"iters\":%d,\"checked_heads\":%ld,"
            "\"delta_hist\":[%ld,%ld,%ld,%ld],\"mean_rel_dev_pct\":%.4f,\"cpu_fp32_seconds\":%.4f,"
            "\"cpu_int8_seconds\":%.4f,\"cpu_threads\":%d,\"cpu_heads_extrapolate_factor\":%.3f,\"pass\":%s}\n",
            c.name.c_str(), c.B, c.H, c.S, Sq, c.d, c.dist.c_str(), c.pad.c_str(), (unsigned long long)opt.seed, us_mean,
            singles.front(), singles[singles.size() / 2], tops, 100 * tops / kInt8PeakTops, opt.iters,
            opt.check ? cpu_heads : 0, hist[0], hist[1], hist[2], hist[3], dev_pct, cpu_fp32_s, cpu_i8_s, threads,
            (double)heads / cpu_heads, pass ? "true" : "false");
  fflush(stdout);
  return pass;
}

}  // namespace

// Quantisation front end / back end (include/fmha_quant.h): parity with inc/utils.hpp:23-39,53 and HBM throughput.
static bool run_quant(long mib, const Options& opt) {
  const long long n = ((long long)mib << 20) / 4 + 3;  // an element count that is not a multiple of four
  std::vector<float> x((size_t)n);
  Rng rng(opt.seed ^ 0x51ull);
  for (long long i = 0; i < n; ++i) x[(size_t)i] = (float)(3.0 * rng.normal());
  x[(size_t)(n / 3)] = -17.25f;  // the maximum, a negative number
  float *dx, *dam, *dback;
  int8_t* dq;
  CHECK_HIP(hipMalloc(&dx, (size_t)n * 4)), CHECK_HIP(hipMalloc(&dback, (size_t)n * 4 + 16));
  CHECK_HIP(hipMalloc(&dq, (size_t)n + 16)), CHECK_HIP(hipMalloc(&dam, 4));
  CHECK_HIP(hipMemcpy(dx, x.data(), (size_t)n * 4, hipMemcpyHostToDevice));
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0)), CHECK_HIP(hipEventCreate(&e1));
  const int iters = opt.iters < 200 ? opt.iters : 200, warm = opt.warmup < 50 ? opt.warmup : 50;
  auto timed = [&](const char* what, double bytes, auto&& call) {
    for (int i = 0; i < warm; ++i) call();
    CHECK_HIP(hipStreamSynchronize(stream));
    CHECK_HIP(hipEventRecord(e0, stream));
    for (int i = 0; i < iters; ++i) call();
    CHECK_HIP(hipEventRecord(e1, stream));
    CHECK_HIP(hipEventSynchronize(e1));
    float ms = 0;
    CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
    const double us = ms * 1e3 / iters, gbs = bytes / us * 1e-3;
    printf("%-28s %10.2f us/call  %8.1f GB/s  %5.1f %% of 8000 GB/s HBM peak  (%.0f algorithmic bytes)\n", what, us, gbs,
           100.0 * gbs / 8000.0, bytes);
  };
  int st = 0;
  timed("FMHAAbsMaxF32", 4.0 * n, [&] { st |= FMHAAbsMaxF32(stream, dx, n, dam); });
  timed("FMHAQuantizeI8 (device amax)", 5.0 * n, [&] { st |= FMHAQuantizeI8(stream, dx, n, 0.f, dam, dq); });
  timed("FMHADequantizeI8", 5.0 * n, [&] { st |= FMHADequantizeI8(stream, dq, n, 17.25f, dback); });
  if (st != FMHA_I8_OK) {
    fprintf(stderr, "quantisation entry points failed: %s\n", FMHAInferI8StatusString(st));
    return false;
  }
  float amax = 0;
  std::vector<int8_t> q((size_t)n);
  std::vector<float> back((size_t)n);
  CHECK_HIP(hipMemcpy(&amax, dam, 4, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(q.data(), dq, (size_t)n, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(back.data(), dback, (size_t)n * 4, hipMemcpyDeviceToHost));
  long long bad_q = 0, bad_d = 0;
  const float want_amax = fmha_oracle::abs_max(x.data(), n);
  for (long long i = 0; i < n; ++i) {
    if (q[(size_t)i] != (int8_t)fmha_oracle::quantize_i8(x[(size_t)i], want_amax)) ++bad_q;
    if (back[(size_t)i] != (float)q[(size_t)i] / 127.0f * 17.25f) ++bad_d;
  }
  bool ok = amax == want_amax && bad_q == 0 && bad_d == 0;
  printf("quantisation parity over %lld elements: amax %g (checker %g), quantise mismatches %lld, de-quantise mismatches "
         "%lld  [%s]\n", n, amax, want_amax, bad_q, bad_d, ok ? "PASS" : "FAIL");

  // the same element count as bfloat16 (the upper halves of the floats above): checked against the widened values
  std::vector<uint16_t> h((size_t)n);
  std::vector<float> wide((size_t)n);
  for (long long i = 0; i < n; ++i) {
    uint32_t u;
    memcpy(&u, &x[(size_t)i], 4);
    h[(size_t)i] = (uint16_t)(u >> 16);
    u &= 0xffff0000u;
    memcpy(&wide[(size_t)i], &u, 4);
  }
  uint16_t* dh = reinterpret_cast<uint16_t*>(dx);        // reuse the float buffers: half the bytes
  uint16_t* dhback = reinterpret_cast<uint16_t*>(dback);
  CHECK_HIP(hipMemcpy(dh, h.data(), (size_t)n * 2, hipMemcpyHostToDevice));
  st = 0;
  timed("FMHAAbsMaxBF16", 2.0 * n, [&] { st |= FMHAAbsMaxBF16(stream, dh, n, dam); });
  timed("FMHAQuantizeI8BF16 (device amax)", 3.0 * n, [&] { st |= FMHAQuantizeI8BF16(stream, dh, n, 0.f, dam, dq); });
  timed("FMHADequantizeI8BF16", 3.0 * n, [&] { st |= FMHADequantizeI8BF16(stream, dq, n, 17.25f, dhback); });
  if (st != FMHA_I8_OK) {
    fprintf(stderr, "bfloat16 quantisation entry points failed: %s\n", FMHAInferI8StatusString(st));
    return false;
  }
  std::vector<uint16_t> hback((size_t)n);
  CHECK_HIP(hipMemcpy(&amax, dam, 4, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(q.data(), dq, (size_t)n, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(hback.data(), dhback, (size_t)n * 2, hipMemcpyDeviceToHost));
  const float want_amax_h = fmha_oracle::abs_max(wide.data(), n);
  bad_q = bad_d = 0;
  for (long long i = 0; i < n; ++i) {
    if (q[(size_t)i] != (int8_t)fmha_oracle::quantize_i8(wide[(size_t)i], want_amax_h)) ++bad_q;
    const float f = (float)q[(size_t)i] / 127.0f * 17.25f;
    uint32_t u;
    memcpy(&u, &f, 4);
    if (hback[(size_t)i] != (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16)) ++bad_d;
  }
  const bool ok_h = amax == want_amax_h && bad_q == 0 && bad_d == 0;
  printf("bfloat16 quantisation parity over %lld elements: amax %g (checker %g), quantise mismatches %lld, de-quantise "
         "mismatches %lld  [%s]\n", n, amax, want_amax_h, bad_q, bad_d, ok_h ? "PASS" : "FAIL");
  ok = ok && ok_h;
  CHECK_HIP(hipFree(dx)), CHECK_HIP(hipFree(dback)), CHECK_HIP(hipFree(dq)), CHECK_HIP(hipFree(dam));
  return ok;
}

int main(int argc, char** argv) {
  Options opt;
  std::vector<Case> cases;
  Case custom;
  bool have_custom = false;
  long calib_mib = 0, quant_mib = 0;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    auto val = [&]() -> const char* {
      if (i + 1 >= argc) {
        fprintf(stderr, "%s needs a value\n", a.c_str());
        exit(2);
      }
      return argv[++i];
    };
    if (a == "--config") cases.push_back(config_case(atoi(val())));
    else if (a == "--sweep") {
      // test_fmha_i8.cpp:295-309: every length of the launch ladder (src/fmha_i8.cu:39-154)
      for (int S : {64, 128, 192, 256, 320, 384, 448, 512, 1024, 2048, 4096})
        for (int d : {64, 128}) {
          Case c;
          c.name = "sweep", c.B = 1, c.H = 1, c.S = S, c.d = d, c.dist = "reference", c.pad = "scatter";
          c.measured_o_amax = true;
          cases.push_back(c);
        }
    } else if (a == "--B") custom.B = atoi(val()), have_custom = true;
    else if (a == "--H") custom.H = atoi(val()), have_custom = true;
    else if (a == "--S") custom.S = atoi(val()), have_custom = true;
    else if (a == "--Sq") custom.Sq = atoi(val()), have_custom = true;
    else if (a == "--d") custom.d = atoi(val()), have_custom = true;
    else if (a == "--valid") custom.valid = atoi(val()), custom.pad = "valid";
    else if (a == "--pad") custom.pad = val();
    else if (a == "--dist") custom.dist = val();
    else if (a == "--seed") opt.seed = strtoull(val(), nullptr, 10);
    else if (a == "--iters") opt.iters = atoi(val());
    else if (a == "--warmup") opt.warmup = atoi(val());
    else if (a == "--cpu-heads") opt.cpu_heads = atol(val());
    else if (a == "--cpu-threads") opt.cpu_threads = atoi(val());
    else if (a == "--no-check") opt.check = false;
    else if (a == "--full-range-p") opt.full_range_p = true;
    else if (a == "--json") opt.json = val();
    else if (a == "--calibrate-copy") calib_mib = atol(val());
    else if (a == "--quant") quant_mib = atol(val());
    else {
      fprintf(stderr, "unknown argument %s\n", a.c_str());
      return 2;
    }
  }
  if (have_custom) {
    custom.name = "custom";
    custom.measured_o_amax = custom.dist == "reference" && (custom.Sq == 0 || custom.Sq == custom.S);
    cases.push_back(custom);
  }
  if (cases.empty()) cases.push_back(config_case(1));
  hipDeviceProp_t prop;
  CHECK_HIP(hipGetDeviceProperties(&prop, 0));
  printf("%s | device %s, %d CUs, %.0f MHz -> CU*8192*clk = %.1f int8 TOPS | host threads %u\n", FMHAInferI8Version(),
         prop.gcnArchName, prop.multiProcessorCount, prop.clockRate / 1e3,
         prop.multiProcessorCount * 8192.0 * prop.clockRate * 1e3 / 1e12, std::thread::hardware_concurrency());
  if (calib_mib > 0) {
    void *src, *dst;
    const size_t bytes = (size_t)calib_mib << 20;
    CHECK_HIP(hipMalloc(&src, bytes)), CHECK_HIP(hipMalloc(&dst, bytes));
    CHECK_HIP(hipMemset(src, 1, bytes));
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipFree(src)), CHECK_HIP(hipFree(dst));
    printf("calibration copy: %ld MiB device to device (reads %zu bytes, writes %zu bytes)\n", calib_mib, bytes, bytes);
  }
  if (quant_mib > 0) {
    const bool ok = run_quant(quant_mib, opt);
    printf("%s\n", ok ? "ALL CASES PASS" : "SOME CASES FAILED");
    return ok ? 0 : 1;
  }
  FILE* json = opt.json.empty() ? nullptr : fopen(opt.json.c_str(), "w");
  bool all = true;
  for (const Case& c : cases) all = run_case(c, opt, json) && all;
  if (json) fclose(json);
  printf("%s\n", all ? "ALL CASES PASS" : "SOME CASES FAILED");
  return all ? 0 : 1;
}
