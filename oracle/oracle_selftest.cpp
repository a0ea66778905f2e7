// TEST INFRASTRUCTURE ONLY.  Runs every function of fmha_oracle.hpp on small and awkward shapes.  Built with
// -fsanitize=address,undefined by `make -C oracle sanitize` (host code only, no GPU): an index of the checker that
// leaves its arrays, a signed overflow or a misaligned access ends the program with a report.  The values are only
// checked where a closed form is at hand - the parity of the checker itself is the business of the test suite.
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "fmha_oracle.hpp"

namespace {

int failures = 0;
void expect(bool ok, const char* what) {
  if (!ok) {
    ++failures;
    fprintf(stderr, "FAILED: %s\n", what);
  }
}

// exact-size buffers (no slack): the sanitizer sees the first byte past any of them
struct Problem {
  int B, H, Sq, S, d;
  std::vector<int8_t> q, k, v, mask, o;
};
Problem make(int B, int H, int Sq, int S, int d, unsigned seed, int masked_from) {
  Problem p{B, H, Sq, S, d, {}, {}, {}, {}, {}};
  std::mt19937 rng(seed);
  std::uniform_int_distribution<int> byte(-127, 127);
  p.q.resize((size_t)B * H * Sq * d), p.k.resize((size_t)B * H * S * d), p.v.resize(p.k.size());
  p.mask.assign((size_t)B * S, 0), p.o.assign(p.q.size(), 99);
  for (auto& x : p.q) x = (int8_t)byte(rng);
  for (auto& x : p.k) x = (int8_t)byte(rng);
  for (auto& x : p.v) x = (int8_t)byte(rng);
  for (int b = 0; b < B; ++b)
    for (int j = 0; j < S; ++j) p.mask[(size_t)b * S + j] = (masked_from >= 0 && j >= masked_from) ? 1 : 0;
  return p;
}

void attention_shapes() {
  const int shapes[][5] = {{1, 1, 1, 1, 64},   {2, 1, 3, 5, 64},     {1, 2, 70, 70, 128}, {1, 1, 64, 64, 64},
                           {1, 1, 33, 129, 64}, {2, 2, 128, 192, 128}, {1, 1, 200, 63, 64}, {1, 1, 256, 256, 128}};
  for (const auto& s : shapes)
    for (int full = 0; full < 2; ++full)
      for (int masked_from : {-1, s[3] / 2 + 1, 0}) {
        Problem p = make(s[0], s[1], s[2], s[3], s[4], 7u + (unsigned)s[3], masked_from);
        const int block = (s[3] + 63) / 64 * 64 % 128 == 0 ? 128 : 64;
        fmha_oracle::fmha_i8_cpu_blockwise_cross(p.q.data(), p.k.data(), p.v.data(), p.mask.data(), p.o.data(), p.B, p.H,
                                                 p.Sq, p.S, p.d, 3.f, 4.f, 2.f, 1.f, block, 2, 0, (long)p.B * p.H,
                                                 full != 0);
        std::vector<int8_t> again(p.o.size(), 11);
        fmha_oracle::fmha_i8_cpu_blockwise_cross(p.q.data(), p.k.data(), p.v.data(), p.mask.data(), again.data(), p.B,
                                                 p.H, p.Sq, p.S, p.d, 3.f, 4.f, 2.f, 1.f, block, 1, 0, (long)p.B * p.H,
                                                 full != 0);
        expect(again == p.o, "the checker is deterministic and independent of the thread count");
        if (masked_from == 0) {
          bool zero = true;
          for (int8_t x : p.o) zero = zero && x == 0;
          expect(zero, "no key left: zeros");
        }
      }
  // uniform attention, both modes: O = rne(v_amax/o_amax * mean V) (here v_amax/o_amax = 1 and V constant: exact)
  for (int full = 0; full < 2; ++full) {
    Problem p = make(1, 1, 40, 100, 64, 3u, 77);
    std::fill(p.q.begin(), p.q.end(), (int8_t)0);
    std::fill(p.v.begin(), p.v.end(), (int8_t)-45);
    fmha_oracle::fmha_i8_cpu_blockwise_cross(p.q.data(), p.k.data(), p.v.data(), p.mask.data(), p.o.data(), 1, 1, 40, 100,
                                             64, 1.f, 1.f, 1.f, 1.f, 64, 2, 0, 1, full != 0);
    bool ok = true;
    for (int8_t x : p.o) ok = ok && x == -45;
    expect(ok, "uniform attention over a constant V returns that constant");
  }
  // self-attention wrapper and the float path
  Problem p = make(2, 2, 128, 128, 64, 5u, 100);
  fmha_oracle::fmha_i8_cpu_blockwise(p.q.data(), p.k.data(), p.v.data(), p.mask.data(), p.o.data(), 2, 2, 128, 64, 1.f, 1.f,
                                     1.f, 1.f, 128, 3, 1, 3);  // heads 1 and 2 only
  std::vector<float> qf(p.q.begin(), p.q.end()), kf(p.k.begin(), p.k.end()), vf(p.v.begin(), p.v.end()), of(p.q.size(), 0.f);
  for (auto& x : qf) x *= 0.01f;
  fmha_oracle::fmha_fp32_cpu(qf.data(), kf.data(), vf.data(), p.mask.data(), of.data(), 2, 2, 128, 64, 2, 0, 4);
  bool finite = true;
  for (float x : of) finite = finite && std::isfinite(x);
  expect(finite, "float path: finite results");
}

void primitives() {
  // cpu_gemm in all four layouts on sizes that are not multiples of anything
  const int M = 5, N = 7, K = 3, batch = 2;
  std::vector<float> a((size_t)batch * M * K), b((size_t)batch * N * K), c((size_t)batch * M * N, 0.f);
  for (size_t i = 0; i < a.size(); ++i) a[i] = (float)(i % 5) - 2.f;
  for (size_t i = 0; i < b.size(); ++i) b[i] = (float)(i % 3) - 1.f;
  for (int ta = 0; ta < 2; ++ta)
    for (int tb = 0; tb < 2; ++tb)
      for (int cm = 0; cm < 2; ++cm)
        fmha_oracle::cpu_gemm<float, float, float, float>(a.data(), b.data(), c.data(), M, N, K, (long)M * K, (long)N * K,
                                                          (long)M * N, batch, 1.f, 0.5f, ta != 0, tb != 0, cm != 0);
  // masked softmax: a row with every key masked, a row with one key
  const int Sq = 3, Sk = 5;
  std::vector<float> s((size_t)Sq * Sk, 1.f), pr((size_t)Sq * Sk, -1.f);
  std::vector<int> m(Sk, 1);
  fmha_oracle::cpu_attention_masked_softmax<float, float>(s.data(), pr.data(), m.data(), 1, Sq, Sk, 1, 64);
  bool zero = true;
  for (float x : pr) zero = zero && x == 0.f;
  expect(zero, "softmax of a fully masked row is zeros");
  m[2] = 0;
  fmha_oracle::cpu_attention_masked_softmax<float, float>(s.data(), pr.data(), m.data(), 1, Sq, Sk, 1, 64);
  expect(pr[2] == 1.f && pr[0] == 0.f, "softmax over one unmasked key");
  // quantiser, abs-max (empty input included), the acceptance metric on a length that is no multiple of 64
  expect(fmha_oracle::quantize_i8(1.f, 1.f) == 127 && fmha_oracle::quantize_i8(-3.f, 1.f) == -127, "quantiser clamps");
  expect(fmha_oracle::abs_max(nullptr, 0) == 0.f, "abs_max of nothing is 0");
  std::vector<float> ref(70, 0.5f);
  std::vector<int8_t> res(70, 64);
  expect(fmha_oracle::mean_rel_deviation_pct(res.data(), ref.data(), 70, 1.f) < 5.f, "deviation metric on 70 elements");
  expect(fmha_oracle::reference_row_scale(64) == 0.125f, "1/sqrt(64)");
}

}  // namespace

int main() {
  primitives();
  attention_shapes();
  if (failures) return 1;
  printf("oracle self-test under the sanitizers: ok\n");
  return 0;
}
