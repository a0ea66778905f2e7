// TEST INFRASTRUCTURE ONLY.  CPU restatement of the reference's attention arithmetic, used as the checker by the
// test-suite, by the smoke test and by the CPU-baseline leg of the benchmark.  Nothing that ships in the GPU
// library includes, links or calls this file.
//
// What is restated, and from where (paths relative to the reference tree):
//   cpu_gemm                      inc/cpuGEMM.hpp:8-31        batched naive GEMM, transA/transB/colMajorC semantics
//   cpu_attention_masked_softmax  inc/cpuSoftmax.hpp:11-51    three-pass masked row softmax with 1/sqrt(d) scaling
//   quantize_i8 / abs_max         inc/utils.hpp:23-39         symmetric int8 quantiser (half-up), max |x|
//   mean_rel_deviation_pct        inc/utils.hpp:59-89         the reference test's acceptance metric (< 20 %)
//   fmha_fp32_cpu                 test_fmha_i8.cpp:141-162    GEMM -> masked softmax -> GEMM on floats
//   fmha_i8_cpu_blockwise         inc/fmha_i8.cuh:71-72,87-117,181-253,298-332
//                                                             the int8 pipeline of the GPU kernel, key block by
//                                                             key block, in the reference's float operation order
//
// Pinning status: cpu_gemm and cpu_attention_masked_softmax are checked against the reference's own headers compiled
// from the reference tree (oracle/_ref) and against closed forms; the quantiser against a known-answer table;
// fmha_i8_cpu_blockwise against closed forms (uniform attention, one-hot attention, block-order invariance, mask
// invariances), against an independent vectorised restatement and against fmha_fp32_cpu / the reference headers
// within the reference's own 20 % criterion.  The reference holds no golden vectors for this path and its GPU
// kernel cannot run here, so no bit-level vector from the reference kernel itself exists.
// The full_range_p mode of fmha_i8_cpu_blockwise_cross (P on 255 steps) restates no reference code - the reference
// only plans that variant (README.md:15,186) - and is pinned by the mathematics alone: the same closed forms and
// invariances, an independent restatement, and its smaller distance to float64 attention.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <thread>
#include <vector>

namespace fmha_oracle {

// ---------------------------------------------------------------------------------------------------------------
// inc/cpuGEMM.hpp:8-31.  C = alpha * op(A) * op(B) + beta * C for `batch_count` problems.
//   trans_a == true  : A is stored [M][K] (element (m,k) at m*K+k);   false: stored [K][M] (k*M+m)
//   trans_b == true  : B is stored [K][N] (element (k,n) at k*N+n);   false: stored [N][K] (n*K+k)
//   col_major_c      : element (m,n) of C at n*M+m, else m*N+n
// beta*C is evaluated even when beta == 0, exactly as in the reference (C must be initialised).
template <typename Compute, typename Scale, typename In, typename Out>
void cpu_gemm(const In* a, const In* b, Out* c, int M, int N, int K, long stride_a, long stride_b, long stride_c,
              int batch_count, Scale alpha, Scale beta, bool trans_a, bool trans_b, bool col_major_c) {
  for (int p = 0; p < batch_count; ++p) {
    const In* pa = a + (long)p * stride_a;
    const In* pb = b + (long)p * stride_b;
    Out* pc = c + (long)p * stride_c;
    for (int m = 0; m < M; ++m) {
      for (int n = 0; n < N; ++n) {
        Compute acc = 0;
        for (int kk = 0; kk < K; ++kk) {
          const In av = trans_a ? pa[(long)m * K + kk] : pa[(long)kk * M + m];
          const In bv = trans_b ? pb[(long)kk * N + n] : pb[(long)n * K + kk];
          acc += static_cast<Compute>(av) * static_cast<Compute>(bv);
        }
        const long at = col_major_c ? (long)n * M + m : (long)m * N + n;
        pc[at] = static_cast<Out>(alpha * static_cast<Compute>(acc) + beta * static_cast<Compute>(pc[at]));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// inc/cpuSoftmax.hpp:11-51.  s, p: [batch, head, seq_q, seq_k]; mask: int [batch, seq_k], a key is masked iff its
// entry == 1 (cpuSoftmax.hpp:24).  Row r belongs to batch r / (seq_q*head_num).  Scale 1/sqrt(head_dim) is applied
// inside.  A row with every key masked yields zeros (its sum is 0 but masked entries are written as 0 directly).
template <typename Compute, typename Data>
void cpu_attention_masked_softmax(const Data* s, Data* p, const int* mask, int batch, int seq_q, int seq_k,
                                  int head_num, int head_dim) {
  const long rows = (long)batch * seq_q * head_num;
  const Compute scale = 1 / std::sqrt(static_cast<Compute>(head_dim));
  for (long r = 0; r < rows; ++r) {
    const Data* srow = s + r * seq_k;
    Data* prow = p + r * seq_k;
    const int* mrow = mask + (r / ((long)seq_q * head_num)) * seq_k;
    Compute top = -std::numeric_limits<Compute>::infinity();
    for (int j = 0; j < seq_k; ++j) {
      const Compute val = (mrow[j] == 1) ? -std::numeric_limits<Compute>::infinity() : static_cast<Compute>(srow[j]);
      top = std::max(val * scale, top);
    }
    Compute denom = 0;
    for (int j = 0; j < seq_k; ++j)
      denom += (mrow[j] == 1) ? static_cast<Compute>(0) : std::exp(static_cast<Compute>(srow[j]) * scale - top);
    for (int j = 0; j < seq_k; ++j)
      prow[j] = (mrow[j] == 1) ? static_cast<Data>(0)
                               : static_cast<Data>(std::exp(static_cast<Compute>(srow[j]) * scale - top) / denom);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// inc/utils.hpp:23-29: scale = 127/amax, floorf(x*scale + 0.5), clamp to [-127, 127].  The 0.5 is a double literal
// there, so the add is exact in double, and floorf takes a float, so the sum is rounded to float before the floor: the
// one float just below 0.5 (0x3EFFFFFF) sums to 1 - 2^-25, rounds to 1.0f and quantises to 1, not 0.
inline int32_t quantize_i8(float x, float amax) {
  const float scale = 127.0f / amax;
  const float scaled = x * scale;
  int32_t q = static_cast<int32_t>(floorf(static_cast<float>(static_cast<double>(scaled) + 0.5)));
  return q < -127 ? -127 : (q > 127 ? 127 : q);
}

// inc/utils.hpp:31-39: max |x|, 0 for an empty range.
inline float abs_max(const float* x, long n) {
  float best = 0.0f;
  for (long i = 0; i < n; ++i) best = std::max(best, std::fabs(x[i]));
  return best;
}

// inc/utils.hpp:59-89: 100/len * sum |res/127*o_amax - ref| / (|ref| + 0.01); the reference asserts < 20.
// The reference accumulates in float over rows of 64 and drops a tail of len % 64 elements; so does this.
inline float mean_rel_deviation_pct(const int8_t* res, const float* ref, long len, float o_amax) {
  float total = 0.0f;
  const long full = (len / 64) * 64;
  for (long i = 0; i < full; ++i) {
    const float deq = static_cast<float>(res[i]) / 127.0f * o_amax;
    const float dev = std::fabs(deq - ref[i]);
    total = static_cast<float>(static_cast<double>(total) + dev / (std::fabs(ref[i]) + 0.01));
  }
  return static_cast<float>(total * 100.0 / len);
}

// ---------------------------------------------------------------------------------------------------------------
// inc/fmha_i8.cuh:13-34,71: the kernel's 1/sqrt(d) is 1.0f / sqrtExpr(d) where sqrtExpr is a Newton iteration
// x_{n+1} = 0.5*(x_n + d/x_n): quotient and sum in float, the halving through a double 0.5, the result rounded back
// to float, stopped at a fixed point.
inline float reference_row_scale(int head_dim) {
  const float x = static_cast<float>(head_dim);
  float cur = x, prev = 0.0f;
  for (int guard = 0; guard < 200 && cur != prev; ++guard) {
    const float next = static_cast<float>(0.5 * static_cast<double>(cur + x / cur));
    prev = cur;
    cur = next;
  }
  return 1.0f / cur;
}

template <typename F>
inline void parallel_for(long n, int threads, F&& body) {
  if (threads <= 1 || n <= 1) {
    for (long i = 0; i < n; ++i) body(i);
    return;
  }
  const int t = (int)std::min<long>(threads, n);
  std::vector<std::thread> pool;
  pool.reserve(t);
  for (int w = 0; w < t; ++w)
    pool.emplace_back([&, w]() {
      for (long i = w; i < n; i += t) body(i);
    });
  for (auto& th : pool) th.join();
}

// ---------------------------------------------------------------------------------------------------------------
// The int8 pipeline of inc/fmha_i8.cuh for ONE (batch, head), all query rows.
//   k, v : int8 [S][d] of this head;  mask: int8 [S] of this batch, nonzero = masked out (fmha_i8.cuh:189-192)
//   q, o : int8 [Sq][d] of this head.  The reference has Sq == S only (one SEQ_LEN sizes everything, fmha_i8.cuh:45);
//          each query row is processed on its own below, as it is in the reference (a warp's 16 rows share nothing
//          but the K/V tiles), so any Sq is the same arithmetic applied to another number of rows.
//   block      : keys per softmax block (BASE_SEQ_LEN: 128, or 64 for the reference's 64-multiples); for a key count
//                that is no multiple of 64 the caller passes the block of the next multiple of 64
// Differences from the reference kernel, both deliberate and both outside what its own test exercises:
//   * a key block with every key masked is skipped (reference: harmless when it is not the first block, NaN when it
//     is, fmha_i8.cuh:91-92,116-117,301-310);
//   * a row with no unmasked key at all yields 0 (as inc/cpuSoftmax.hpp:18-47 does).
inline void fmha_i8_head_blockwise(const int8_t* q, const int8_t* k, const int8_t* v, const int8_t* mask, int8_t* o,
                                   int Sq, int S, int d, float q_amax, float k_amax, float v_amax, float o_amax,
                                   int block, bool full_range_p = false) {
  const float row_scale = reference_row_scale(d);                    // fmha_i8.cuh:71
  const float scale_qk_out = q_amax * k_amax / (127.f * 127.f);      // fmha_i8.cuh:72
  // full_range_p: the "uint8 x int8" variant that the reference plans and does not have (README.md:15,186): P keeps
  // all 255 steps of a byte, P = rne(255 p) in [0, 255], and every 128 of the pipeline becomes 255.
  const float p_scale = full_range_p ? 255.f : -128.f;               // fmha_i8.cuh:241
  const float scale_v_out = v_amax * (1.0f / (o_amax * std::fabs(p_scale)));  // fmha_i8.cuh:318
  const int kMaskedInt = static_cast<int>(-1e6);                     // fmha_i8.cuh:191-192
  std::vector<int32_t> s_int(block);
  std::vector<float> p_f(block);
  std::vector<int32_t> p_i8(block);
  std::vector<int32_t> o_tilde(d);
  std::vector<float> o_f(d);
  for (int i = 0; i < Sq; ++i) {
    float m_old = -1e6f, l_old = 0.0f;                                // fmha_i8.cuh:91-92
    std::fill(o_f.begin(), o_f.end(), 0.0f);                          // fmha_i8.cuh:105-108
    const int8_t* qi = q + (long)i * d;
    for (int k0 = 0; k0 < S; k0 += block) {
      const int nb = std::min(block, S - k0);
      bool any_valid = false;
      for (int j = 0; j < nb; ++j) any_valid |= (mask[k0 + j] == 0);
      if (!any_valid) continue;
      // GEMM 1 (fmha_i8.cuh:120-172): exact int32 dot products.
      for (int j = 0; j < nb; ++j) {
        const int8_t* kj = k + (long)(k0 + j) * d;
        int32_t acc = 0;
        for (int c = 0; c < d; ++c) acc += (int32_t)qi[c] * (int32_t)kj[c];
        s_int[j] = acc;
      }
      // Block-local row max (fmha_i8.cuh:116,181-206): masked keys enter as the integer -1000000; the max starts
      // at -1e6f; value = (row_scale * float(int)) * scale_qk_out, which is monotone in the integer.
      // A last block that is only partly there (a key count that is no multiple of the block; the reference has no
      // such length, src/fmha_i8.cu:39-154) is a full block whose missing keys are masked: they enter the maximum too.
      int top_int = nb < block ? kMaskedInt : std::numeric_limits<int>::min();
      for (int j = 0; j < nb; ++j) top_int = std::max(top_int, mask[k0 + j] ? kMaskedInt : s_int[j]);
      const float m_blk = std::max(-1e6f, row_scale * static_cast<float>(top_int) * scale_qk_out);
      // exp and un-quantised row sum (fmha_i8.cuh:208-235); a*b - c contracts to one fma under nvcc's default.
      float l_blk = 0.0f;
      for (int j = 0; j < nb; ++j) {
        const float e = std::exp(std::fma(row_scale * static_cast<float>(s_int[j]), scale_qk_out, -m_blk));
        p_f[j] = mask[k0 + j] ? 0.0f : e;
        l_blk += p_f[j];
      }
      // P -> int8 in [-128, 0], round-half-even (fmha_i8.cuh:241,249); full range: a byte in [0, 255].
      for (int j = 0; j < nb; ++j)
        p_i8[j] = full_range_p ? (int32_t)std::nearbyint(std::max(std::min(255.f * p_f[j], 255.f), 0.f))
                               : (int32_t)std::nearbyint(std::max(std::min(-128.f * p_f[j], 0.f), -128.f));
      // GEMM 2 (fmha_i8.cuh:255-296): exact int32.
      std::fill(o_tilde.begin(), o_tilde.end(), 0);
      for (int j = 0; j < nb; ++j) {
        const int32_t pj = p_i8[j];
        if (pj == 0) continue;
        const int8_t* vj = v + (long)(k0 + j) * d;
        for (int c = 0; c < d; ++c) o_tilde[c] += pj * (int32_t)vj[c];
      }
      // Online merge, O kept normalised (fmha_i8.cuh:298-315).
      const float m_new = std::max(m_old, m_blk);
      const float a = std::exp(m_old - m_new);
      const float bb = std::exp(m_blk - m_new);
      const float l_new = a * l_old + bb * l_blk;
      const float inv = 1.0f / l_new;
      const float keep = l_old * a;
      const float p_sign = full_range_p ? 1.f : -1.f;
      for (int c = 0; c < d; ++c) o_f[c] = inv * (keep * o_f[c] + bb * (p_sign * static_cast<float>(o_tilde[c])));
      l_old = l_new;
      m_old = m_new;
    }
    // Epilogue (fmha_i8.cuh:318-332).
    int8_t* oi = o + (long)i * d;
    for (int c = 0; c < d; ++c) {
      const float y = std::max(std::min(scale_v_out * o_f[c], 127.f), -127.f);
      oi[c] = (l_old > 0.0f) ? (int8_t)std::nearbyint(y) : (int8_t)0;
    }
  }
}

// All heads in [head_begin, head_end) of the flattened (batch*head_num) index; others are left untouched in `o`.
// q, o: [B][H][Sq][d]; k, v: [B][H][S][d]; mask: [B][S].
inline void fmha_i8_cpu_blockwise_cross(const int8_t* q, const int8_t* k, const int8_t* v, const int8_t* mask,
                                        int8_t* o, int B, int H, int Sq, int S, int d, float q_amax, float k_amax,
                                        float v_amax, float o_amax, int block, int threads, long head_begin,
                                        long head_end, bool full_range_p = false) {
  const long hd_q = (long)Sq * d, hd = (long)S * d;
  head_begin = std::max<long>(head_begin, 0);
  head_end = std::min<long>(head_end, (long)B * H);
  parallel_for(head_end - head_begin, threads, [&](long t) {
    const long bh = head_begin + t;
    const long b = bh / H;
    fmha_i8_head_blockwise(q + bh * hd_q, k + bh * hd, v + bh * hd, mask + b * S, o + bh * hd_q, Sq, S, d, q_amax,
                           k_amax, v_amax, o_amax, block, full_range_p);
  });
}
inline void fmha_i8_cpu_blockwise(const int8_t* q, const int8_t* k, const int8_t* v, const int8_t* mask, int8_t* o,
                                  int B, int H, int S, int d, float q_amax, float k_amax, float v_amax, float o_amax,
                                  int block, int threads, long head_begin, long head_end) {
  fmha_i8_cpu_blockwise_cross(q, k, v, mask, o, B, H, S, S, d, q_amax, k_amax, v_amax, o_amax, block, threads,
                              head_begin, head_end);
}

// ---------------------------------------------------------------------------------------------------------------
// test_fmha_i8.cpp:141-162 evaluated head by head (the B*H*S*S float buffers are never materialised):
// S = Q.K^T (cpu_gemm, T/N, row-major C), P = masked softmax, O = P.V (cpu_gemm, T/T, row-major C).
// mask: int8 [B][S], nonzero = masked (converted to the int {0,1} array the softmax expects).
inline void fmha_fp32_cpu(const float* q, const float* k, const float* v, const int8_t* mask, float* o, int B, int H,
                          int S, int d, int threads, long head_begin, long head_end) {
  const long hd = (long)S * d;
  head_begin = std::max<long>(head_begin, 0);
  head_end = std::min<long>(head_end, (long)B * H);
  parallel_for(head_end - head_begin, threads, [&](long t) {
    const long bh = head_begin + t;
    const long b = bh / H;
    std::vector<float> s((long)S * S, 0.0f), p((long)S * S, 0.0f);
    std::vector<int> m(S);
    for (int j = 0; j < S; ++j) m[j] = mask[b * S + j] ? 1 : 0;
    cpu_gemm<float, float, float, float>(q + bh * hd, k + bh * hd, s.data(), S, S, d, 0, 0, 0, 1, 1.0f, 0.0f, true,
                                         false, false);
    cpu_attention_masked_softmax<float, float>(s.data(), p.data(), m.data(), 1, S, S, 1, d);
    float* oh = o + bh * hd;
    std::fill(oh, oh + hd, 0.0f);
    cpu_gemm<float, float, float, float>(p.data(), v + bh * hd, oh, S, d, S, 0, 0, 0, 1, 1.0f, 0.0f, true, true,
                                         false);
  });
}

}  // namespace fmha_oracle
