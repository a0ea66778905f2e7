// TEST INFRASTRUCTURE ONLY.  Compiles the REFERENCE's own CPU templates, from the headers where they lie in the
// reference tree (-I<reference>/inc), into oracle/_ref/libfmha_ref_cpu.so.  Nothing of the reference is copied
// into this repository: this file only names the two headers and instantiates what test_fmha_i8.cpp instantiates.
// <algorithm> and <iostream> come first because cpuSoftmax.hpp uses max() through `using namespace std` without
// including <algorithm> itself.  inc/utils.hpp is not included: it needs <cuda.h>, which this image lacks.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <iostream>
#include <vector>
#include "cpuGEMM.hpp"
#include "cpuSoftmax.hpp"

extern "C" {

// cpuGEMM<float,float,float,float> (test_fmha_i8.cpp:144-147,156-159).
void ref_cpu_gemm_f32(float* a, float* b, float* c, int M, int N, int K, int sa, int sb, int sc, int batch,
                      float alpha, float beta, int trans_a, int trans_b, int col_major_c) {
  cpuGEMM<float, float, float, float>(a, b, c, M, N, K, sa, sb, sc, batch, alpha, beta, trans_a != 0, trans_b != 0,
                                      nullptr, col_major_c != 0);
}
// cpuGEMM<int32_t,int32_t,int8_t,int32_t>: the template instantiated on the int8 pipeline's types.
void ref_cpu_gemm_i8(int8_t* a, int8_t* b, int32_t* c, int M, int N, int K, int sa, int sb, int sc, int batch,
                     int alpha, int beta, int trans_a, int trans_b, int col_major_c) {
  cpuGEMM<int32_t, int32_t, int8_t, int32_t>(a, b, c, M, N, K, sa, sb, sc, batch, alpha, beta, trans_a != 0,
                                             trans_b != 0, nullptr, col_major_c != 0);
}
// cpuAttentionMaskedSoftmax<float,float> (test_fmha_i8.cpp:149-150).
void ref_cpu_attention_masked_softmax_f32(float* s, float* p, const int* mask, int batch, int seq_q, int seq_k,
                                          int head_num, int head_dim) {
  cpuAttentionMaskedSoftmax<float, float>(s, p, mask, batch, seq_q, seq_k, head_num, head_dim);
}
// The reference test's CPU path for heads [head_begin, head_end) (test_fmha_i8.cpp:141-162), one head at a time so
// that the S and P buffers stay S*S floats.  mask: int [B][S], 1 = masked.
void ref_fmha_fp32_heads(float* q, float* k, float* v, const int* mask, float* o, int B, int H, int S, int d,
                         long head_begin, long head_end) {
  std::vector<float> s((size_t)S * S), p((size_t)S * S);
  const long hd = (long)S * d;
  for (long bh = head_begin; bh < head_end && bh < (long)B * H; ++bh) {
    std::fill(s.begin(), s.end(), 0.0f);
    std::fill(p.begin(), p.end(), 0.0f);
    std::fill(o + bh * hd, o + (bh + 1) * hd, 0.0f);
    cpuGEMM<float, float, float, float>(q + bh * hd, k + bh * hd, s.data(), S, S, d, 0, 0, 0, 1, 1.0f, 0.0f, GEMM_OP_T,
                                        GEMM_OP_N, nullptr, false);
    cpuAttentionMaskedSoftmax<float, float>(s.data(), p.data(), mask + (bh / H) * S, 1, S, S, 1, d);
    cpuGEMM<float, float, float, float>(p.data(), v + bh * hd, o + bh * hd, S, d, S, 0, 0, 0, 1, 1.0f, 0.0f, GEMM_OP_T,
                                        GEMM_OP_T, nullptr, false);
  }
}

}  // extern "C"
