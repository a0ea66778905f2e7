// TEST INFRASTRUCTURE ONLY.  extern "C" face of fmha_oracle.hpp so that the Python tests (ctypes) and the C++ test
// harness can call the CPU checker.  The GPU library never links this.
#include "fmha_oracle.hpp"

using namespace fmha_oracle;

extern "C" {

// inc/cpuGEMM.hpp:8-31 instantiated <float,float,float,float> (the only instantiation the reference uses,
// test_fmha_i8.cpp:144,156) and <int32,int32,int8,int32> (the int8 pipeline's GEMMs).
void oracle_cpu_gemm_f32(const float* a, const float* b, float* c, int M, int N, int K, long sa, long sb, long sc,
                         int batch, float alpha, float beta, int trans_a, int trans_b, int col_major_c) {
  cpu_gemm<float, float, float, float>(a, b, c, M, N, K, sa, sb, sc, batch, alpha, beta, trans_a != 0, trans_b != 0,
                                       col_major_c != 0);
}
void oracle_cpu_gemm_i8(const int8_t* a, const int8_t* b, int32_t* c, int M, int N, int K, long sa, long sb, long sc,
                        int batch, int alpha, int beta, int trans_a, int trans_b, int col_major_c) {
  cpu_gemm<int32_t, int32_t, int8_t, int32_t>(a, b, c, M, N, K, sa, sb, sc, batch, alpha, beta, trans_a != 0,
                                              trans_b != 0, col_major_c != 0);
}
// inc/cpuSoftmax.hpp:11-51 <float,float>.
void oracle_cpu_attention_masked_softmax_f32(const float* s, float* p, const int* mask, int batch, int seq_q,
                                             int seq_k, int head_num, int head_dim) {
  cpu_attention_masked_softmax<float, float>(s, p, mask, batch, seq_q, seq_k, head_num, head_dim);
}
// inc/utils.hpp:23-39,59-89.
void oracle_quantize_i8(const float* x, int8_t* out, long n, float amax) {
  for (long i = 0; i < n; ++i) out[i] = (int8_t)quantize_i8(x[i], amax);
}
float oracle_abs_max(const float* x, long n) { return abs_max(x, n); }
float oracle_mean_rel_deviation_pct(const int8_t* res, const float* ref, long len, float o_amax) {
  return mean_rel_deviation_pct(res, ref, len, o_amax);
}
float oracle_reference_row_scale(int head_dim) { return reference_row_scale(head_dim); }

// inc/fmha_i8.cuh int8 pipeline, heads [head_begin, head_end) of the flattened batch*head index.
void oracle_fmha_i8_blockwise(const int8_t* q, const int8_t* k, const int8_t* v, const int8_t* mask, int8_t* o, int B,
                              int H, int S, int d, float q_amax, float k_amax, float v_amax, float o_amax, int block,
                              int threads, long head_begin, long head_end) {
  fmha_i8_cpu_blockwise(q, k, v, mask, o, B, H, S, d, q_amax, k_amax, v_amax, o_amax, block, threads, head_begin,
                        head_end);
}
// The same pipeline with Sq query rows over S keys (README.md:13 lists it as planned; the rows are independent).
void oracle_fmha_i8_blockwise_cross(const int8_t* q, const int8_t* k, const int8_t* v, const int8_t* mask, int8_t* o,
                                    int B, int H, int Sq, int S, int d, float q_amax, float k_amax, float v_amax,
                                    float o_amax, int block, int threads, long head_begin, long head_end) {
  fmha_i8_cpu_blockwise_cross(q, k, v, mask, o, B, H, Sq, S, d, q_amax, k_amax, v_amax, o_amax, block, threads,
                              head_begin, head_end);
}
// ... and with P on all 255 steps of a byte (README.md:15,186 plans it as "uint8 x int8"; the reference has no code for it).
void oracle_fmha_i8_blockwise_cross_full_range_p(const int8_t* q, const int8_t* k, const int8_t* v, const int8_t* mask,
                                                 int8_t* o, int B, int H, int Sq, int S, int d, float q_amax,
                                                 float k_amax, float v_amax, float o_amax, int block, int threads,
                                                 long head_begin, long head_end) {
  fmha_i8_cpu_blockwise_cross(q, k, v, mask, o, B, H, Sq, S, d, q_amax, k_amax, v_amax, o_amax, block, threads,
                              head_begin, head_end, true);
}
// test_fmha_i8.cpp:141-162 float path.
void oracle_fmha_fp32(const float* q, const float* k, const float* v, const int8_t* mask, float* o, int B, int H, int S,
                      int d, int threads, long head_begin, long head_end) {
  fmha_fp32_cpu(q, k, v, mask, o, B, H, S, d, threads, head_begin, head_end);
}
int oracle_hardware_threads(void) { return (int)std::thread::hardware_concurrency(); }

}  // extern "C"
