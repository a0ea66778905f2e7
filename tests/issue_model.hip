// How a gfx950 SIMD issues vector instructions from the wavefronts that share it (test tool).
//
// The attention kernel is bound by instruction issue, not by the matrix pipe or by memory, so what the SIMD can and
// cannot issue together decides how far any schedule can go.  This program measures it with streams of one
// instruction each (eight independent register chains, inline assembly so that nothing is rescheduled): wavefront
// group 0 (wavefronts 0..3 of a 512-thread workgroup, one per SIMD) runs stream X, group 1 stream Y, a third group an
// MFMA stream.  Output: cycles at 2.4 GHz per instruction PAIR (one instruction of X and one of Y); about 4.3 means
// the two issue together, about 8.5 means one after the other.  It also measures what instruction ALIGNMENT costs: a
// 64-bit-encoded VALU instruction at an address that is 4 mod 8 takes 5.4 to 5.7 cycles instead of 4.7.
//
//     tests/bin/issue_model
//     tests/bin/issue_model --launch-overhead     (a second table: what an empty launch of the kernel's shape costs)
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define CHECK(x)                                                                     \
  do {                                                                               \
    hipError_t e_ = (x);                                                             \
    if (e_ != hipSuccess) {                                                          \
      fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      exit(1);                                                                       \
    }                                                                                \
  } while (0)

// eight instructions over eight independent chains v64..v71; operands v100 = 1.0, v101 = 0, v102 / s21 = byte selector
#define R8(OP) OP(64) OP(65) OP(66) OP(67) OP(68) OP(69) OP(70) OP(71)
#define R192(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) \
                 R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP) R8(OP)
#define S_(x) #x
#define OP_ADD(r) "v_add_f32_e32 v" S_(r) ", v" S_(r) ", v101\n\t"
#define OP_ADD_S(r) "v_add_f32_e32 v" S_(r) ", s20, v" S_(r) "\n\t"
#define OP_MUL(r) "v_mul_f32_e32 v" S_(r) ", v" S_(r) ", v100\n\t"
#define OP_FMA(r) "v_fma_f32 v" S_(r) ", v" S_(r) ", v100, v101\n\t"
#define OP_FMA_S(r) "v_fma_f32 v" S_(r) ", v" S_(r) ", s20, v101\n\t"
#define OP_FMAC(r) "v_fmac_f32_e32 v" S_(r) ", v100, v101\n\t"
#define OP_MOV(r) "v_mov_b32_e32 v" S_(r) ", v101\n\t"
#define OP_MAX3(r) "v_max3_i32 v" S_(r) ", v" S_(r) ", v100, v101\n\t"
#define OP_MAXF(r) "v_max_f32_e32 v" S_(r) ", v" S_(r) ", v101\n\t"
#define OP_PKNORM(r) "v_cvt_pknorm_i16_f32 v" S_(r) ", v" S_(r) ", v101\n\t"
#define OP_PERM(r) "v_perm_b32 v" S_(r) ", v" S_(r) ", v101, v102\n\t"
#define OP_CVT(r) "v_cvt_f32_i32_e32 v" S_(r) ", v" S_(r) "\n\t"
#define OP_EXP(r) "v_exp_f32_e32 v" S_(r) ", v" S_(r) "\n\t"
#define OP_EXPH(r) "v_exp_f16_e32 v" S_(r) ", v" S_(r) "\n\t"
// the half-precision softmax tail: pack-convert, mixed-precision fma with a half result, dot product of two half pairs
#define OP_CVTPKH(r) "v_cvt_pk_f16_f32 v" S_(r) ", v" S_(r) ", v101\n\t"
#define OP_FMAMIX(r) "v_fma_mixlo_f16 v" S_(r) ", v" S_(r) ", v100, v101\n\t"
#define OP_DOT2(r) "v_dot2c_f32_f16_e32 v" S_(r) ", v100, v101\n\t"
// 32 MFMAs per 192 slots (two alternating accumulator tiles): the matrix pipe is then busy all the time
#define MF_(a) "v_mfma_i32_32x32x32_i8 v[" S_(a) ":" S_(a) "+15], v[104:107], v[108:111], v[" S_(a) ":" S_(a) "+15]\n\t"
#define MF4 MF_(0) MF_(16) MF_(0) MF_(16)
#define MF32 MF4 MF4 MF4 MF4 MF4 MF4 MF4 MF4
// 48 half-precision MFMAs of 16 cycles per 192 slots (four alternating accumulator tiles of four registers)
#define MH_(a) "v_mfma_f32_16x16x32_f16 v[" S_(a) ":" S_(a) "+3], v[104:107], v[108:111], v[" S_(a) ":" S_(a) "+3]\n\t"
#define MH4 MH_(0) MH_(4) MH_(8) MH_(12)
#define MH48 MH4 MH4 MH4 MH4 MH4 MH4 MH4 MH4 MH4 MH4 MH4 MH4
// the row sum of the attention kernel on the matrix pipe: four pack-converts, then one half-precision MFMA, 32 times
#define CV4M_(a) "v_cvt_pk_f16_f32 v64, v65, v101\n\tv_cvt_pk_f16_f32 v66, v67, v101\n\tv_cvt_pk_f16_f32 v68, v69, v101\n\tv_cvt_pk_f16_f32 v70, v71, v101\n\t" MH_(a)
#define CV4M4 CV4M_(0) CV4M_(0) CV4M_(0) CV4M_(0)
#define CV4M32 CV4M4 CV4M4 CV4M4 CV4M4 CV4M4 CV4M4 CV4M4 CV4M4

enum Op { kNone, kAdd, kAddS, kMul, kFma, kFmaS, kFmac, kMov, kMax3, kMaxF, kPknorm, kPerm, kCvt, kExp, kExpH, kMfma, kFmaMis, kPknormMis, kAddMis, kMfmaMis,
          kCvtPkH, kFmaMix, kDot2, kMfmaH, kCvtMfmaH };
#define CLOBBER "memory", "s20", "s21", "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", "v10", "v11", "v12", "v13", \
    "v14", "v15", "v16", "v17", "v18", "v19", "v20", "v21", "v22", "v23", "v24", "v25", "v26", "v27", "v28", "v29", "v30",     \
    "v31", "v64", "v65", "v66", "v67", "v68", "v69", "v70", "v71", "v100", "v101", "v102", "v104", "v105", "v106", "v107",   \
    "v108", "v109", "v110", "v111"

// Every stream starts at an 8-byte-aligned address (the compiler aligns nothing inside a function); the "at 4 mod 8"
// variants start one dword later, so that every 64-bit-encoded instruction of the stream straddles an aligned pair.
#define AL ".p2align 3\n\t"
#define MIS ".p2align 3\n\ts_nop 0\n\t"
template <int OP>
__device__ __forceinline__ void stream() {
  if (OP == kFmaMis) asm volatile(MIS R192(OP_FMA) ::: CLOBBER);
  if (OP == kPknormMis) asm volatile(MIS R192(OP_PKNORM) ::: CLOBBER);
  if (OP == kAddMis) asm volatile(MIS R192(OP_ADD) ::: CLOBBER);
  if (OP == kMfmaMis) asm volatile(MIS MF32 ::: CLOBBER);
  if (OP == kAdd) asm volatile(AL R192(OP_ADD) ::: CLOBBER);
  if (OP == kAddS) asm volatile(AL R192(OP_ADD_S) ::: CLOBBER);
  if (OP == kMul) asm volatile(AL R192(OP_MUL) ::: CLOBBER);
  if (OP == kFma) asm volatile(AL R192(OP_FMA) ::: CLOBBER);
  if (OP == kFmaS) asm volatile(AL R192(OP_FMA_S) ::: CLOBBER);
  if (OP == kFmac) asm volatile(AL R192(OP_FMAC) ::: CLOBBER);
  if (OP == kMov) asm volatile(AL R192(OP_MOV) ::: CLOBBER);
  if (OP == kMax3) asm volatile(AL R192(OP_MAX3) ::: CLOBBER);
  if (OP == kMaxF) asm volatile(AL R192(OP_MAXF) ::: CLOBBER);
  if (OP == kPknorm) asm volatile(AL R192(OP_PKNORM) ::: CLOBBER);
  if (OP == kPerm) asm volatile(AL R192(OP_PERM) ::: CLOBBER);
  if (OP == kCvt) asm volatile(AL R192(OP_CVT) ::: CLOBBER);
  if (OP == kExp) asm volatile(AL R192(OP_EXP) ::: CLOBBER);
  if (OP == kExpH) asm volatile(AL R192(OP_EXPH) ::: CLOBBER);
  if (OP == kMfma) asm volatile(AL MF32 ::: CLOBBER);
  if (OP == kCvtPkH) asm volatile(AL R192(OP_CVTPKH) ::: CLOBBER);
  if (OP == kFmaMix) asm volatile(AL R192(OP_FMAMIX) ::: CLOBBER);
  if (OP == kDot2) asm volatile(AL R192(OP_DOT2) ::: CLOBBER);
  if (OP == kMfmaH) asm volatile(AL MH48 ::: CLOBBER);
  if (OP == kCvtMfmaH) asm volatile(AL CV4M32 ::: CLOBBER);  // (160 instructions, not 192: see the row's label)
}

// wavefront group g (256 threads each: one wavefront per SIMD) runs stream X (g = 0), Y (g = 1), Z (g = 2)
template <int X, int Y, int Z>
__global__ __launch_bounds__(768) void issue_streams(int* out, int iters) {
  asm volatile("v_mov_b32 v100, 1.0\n\tv_mov_b32 v101, 0\n\tv_mov_b32 v102, 0x06040200\n\ts_mov_b32 s20, 1.0\n\ts_mov_b32 s21, 0x06040200" ::: CLOBBER);
  const int g = __builtin_amdgcn_readfirstlane(threadIdx.x >> 8);
  if (g == 0) {
    for (int it = 0; it < iters; ++it) stream<X>();
  } else if (g == 1) {
    for (int it = 0; it < iters; ++it) stream<Y>();
  } else {
    for (int it = 0; it < iters; ++it) stream<Z>();
  }
  if (iters < 0) out[0] = 1;
}

template <int X, int Y, int Z>
double cycles_per_pair(int* out, int iters) {
  const int groups = Z != kNone ? 3 : (Y != kNone ? 2 : 1);
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  hipLaunchKernelGGL((issue_streams<X, Y, Z>), dim3(256), dim3(256 * groups), 0, 0, out, iters);
  CHECK(hipDeviceSynchronize());
  double best = 1e30;
  for (int rep = 0; rep < 3; ++rep) {
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL((issue_streams<X, Y, Z>), dim3(256), dim3(256 * groups), 0, 0, out, iters);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    if (ms < best) best = ms;
  }
  return best * 1e-3 * 2.4e9 / ((double)iters * 192.0);
}
#define ROW(X, Y, Z, text) printf("%-58s %6.2f\n", text, cycles_per_pair<X, Y, Z>(out, iters))

// ---- launch overhead: what a launch of the attention kernel's SHAPE costs before it computes anything -------------
// An empty kernel with a given static LDS size, workgroup width and register allocation (a write to the highest
// register makes the allocation what the attention kernel's is), launched back to back on one stream: microseconds
// from launch to launch.
template <int LDS_BYTES, int THREADS, int VGPRS>
__global__ __launch_bounds__(THREADS) void empty_kernel(int* out, int never) {
  __shared__ int lds[LDS_BYTES >= 4 ? LDS_BYTES / 4 : 1];
  if (VGPRS > 128) asm volatile("v_mov_b32 v255, 0" ::: "v255");
  else if (VGPRS > 64) asm volatile("v_mov_b32 v127, 0" ::: "v127");
  if (never) {  // (never true: keeps the LDS array allocated)
    lds[threadIdx.x] = never;
    __syncthreads();
    out[threadIdx.x] = lds[threadIdx.x ^ 1];
  }
}
template <int LDS_BYTES, int THREADS, int VGPRS>
void launch_row(int* out) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  printf("%9d %8d %6d", LDS_BYTES, THREADS, VGPRS);
  for (int grid : {256, 512, 2048}) {
    for (int i = 0; i < 3000; ++i) hipLaunchKernelGGL((empty_kernel<LDS_BYTES, THREADS, VGPRS>), dim3(grid), dim3(THREADS), 0, 0, out, 0);
    CHECK(hipDeviceSynchronize());
    double best = 1e30;
    for (int rep = 0; rep < 3; ++rep) {
      const int calls = 4000;
      CHECK(hipEventRecord(e0));
      for (int i = 0; i < calls; ++i) hipLaunchKernelGGL((empty_kernel<LDS_BYTES, THREADS, VGPRS>), dim3(grid), dim3(THREADS), 0, 0, out, 0);
      CHECK(hipEventRecord(e1));
      CHECK(hipEventSynchronize(e1));
      float ms;
      CHECK(hipEventElapsedTime(&ms, e0, e1));
      if (ms * 1e3 / calls < best) best = ms * 1e3 / calls;
    }
    printf(" %10.2f", best);
  }
  printf("\n");
  CHECK(hipGetLastError());
}
int launch_overhead() {
  int* out;
  CHECK(hipMalloc(&out, 4096));
  printf("# microseconds from launch to launch of an EMPTY kernel, back to back on one stream\n");
  printf("# LDS bytes  threads  VGPRs   grid 256   grid 512  grid 2048\n");
  launch_row<0, 256, 64>(out);
  launch_row<0, 512, 64>(out);
  launch_row<0, 256, 256>(out);
  launch_row<0, 512, 256>(out);
  launch_row<65536, 256, 64>(out);
  launch_row<65536, 512, 64>(out);
  launch_row<65536, 256, 256>(out);
  launch_row<65536, 512, 256>(out);
  launch_row<140288, 256, 64>(out);
  launch_row<140288, 512, 64>(out);
  launch_row<140288, 256, 256>(out);
  launch_row<140288, 512, 256>(out);
  launch_row<140288, 512, 128>(out);
  launch_row<75776, 512, 192>(out);   // the d = 64 kernel
  return 0;
}

int main(int argc, char** argv) {
  if (argc > 1 && !strcmp(argv[1], "--launch-overhead")) return launch_overhead();
  const int iters = argc > 1 ? atoi(argv[1]) : 1000;
  int* out;
  CHECK(hipMalloc(&out, 256));
  for (int warm = 0; warm < 30; ++warm) hipLaunchKernelGGL((issue_streams<kAdd, kAdd, kNone>), dim3(256), dim3(512), 0, 0, out, 2000);
  CHECK(hipDeviceSynchronize());
  printf("# cycles at 2.4 GHz per instruction of each stream (one instruction of every stream counts as one step)\n");
  printf("# -- one wavefront per SIMD: the rate one wavefront can issue at\n");
  ROW(kAdd, kNone, kNone, "v_add_f32 alone");
  ROW(kFma, kNone, kNone, "v_fma_f32 alone");
  ROW(kMax3, kNone, kNone, "v_max3_i32 alone");
  ROW(kExp, kNone, kNone, "v_exp_f32 alone");
  ROW(kExpH, kNone, kNone, "v_exp_f16 alone");
  printf("# -- the same from an address that is 4 mod 8: a 64-bit encoding then straddles two aligned dword pairs\n");
  ROW(kAddMis, kNone, kNone, "v_add_f32 (32-bit encoding) alone, at 4 mod 8");
  ROW(kFmaMis, kNone, kNone, "v_fma_f32 (64-bit encoding) alone, at 4 mod 8");
  ROW(kPknormMis, kNone, kNone, "v_cvt_pknorm_i16_f32 (64-bit) alone, at 4 mod 8");
  ROW(kFmaMis, kFmaMis, kNone, "v_fma_f32 | v_fma_f32, both at 4 mod 8");
  ROW(kMfmaMis, kNone, kNone, "v_mfma_i32_32x32x32_i8 alone, at 4 mod 8 (x 6)");
  printf("# -- two wavefronts per SIMD, plain fp32 arithmetic in both: they issue together\n");
  ROW(kAdd, kAdd, kNone, "v_add_f32 | v_add_f32");
  ROW(kMul, kAdd, kNone, "v_mul_f32 | v_add_f32");
  ROW(kFmac, kAdd, kNone, "v_fmac_f32 | v_add_f32");
  ROW(kFma, kFma, kNone, "v_fma_f32 | v_fma_f32 (64-bit encoding)");
  ROW(kMov, kAdd, kNone, "v_mov_b32 | v_add_f32");
  printf("# -- plain fp32 arithmetic beside integer / conversion / permute: they issue together\n");
  ROW(kAdd, kMax3, kNone, "v_add_f32 | v_max3_i32");
  ROW(kFmac, kPknorm, kNone, "v_fmac_f32 | v_cvt_pknorm_i16_f32");
  ROW(kAdd, kPerm, kNone, "v_add_f32 | v_perm_b32");
  ROW(kAdd, kCvt, kNone, "v_add_f32 | v_cvt_f32_i32");
  printf("# -- integer / conversion / permute / float max in both: one after the other\n");
  ROW(kMax3, kMax3, kNone, "v_max3_i32 | v_max3_i32");
  ROW(kMax3, kPknorm, kNone, "v_max3_i32 | v_cvt_pknorm_i16_f32");
  ROW(kPerm, kPknorm, kNone, "v_perm_b32 | v_cvt_pknorm_i16_f32");
  ROW(kMaxF, kMaxF, kNone, "v_max_f32 | v_max_f32");
  ROW(kCvt, kCvt, kNone, "v_cvt_f32_i32 | v_cvt_f32_i32");
  printf("# -- an SGPR operand in both: one after the other (one constant bus)\n");
  ROW(kAddS, kAdd, kNone, "v_add_f32 (SGPR operand) | v_add_f32");
  ROW(kAddS, kAddS, kNone, "v_add_f32 (SGPR operand) | v_add_f32 (SGPR operand)");
  ROW(kFmaS, kFmaS, kNone, "v_fma_f32 (SGPR operand) | v_fma_f32 (SGPR operand)");
  printf("# -- the exponential: nothing issues beside it\n");
  ROW(kExp, kExp, kNone, "v_exp_f32 | v_exp_f32");
  ROW(kExp, kAdd, kNone, "v_exp_f32 | v_add_f32");
  ROW(kExp, kPknorm, kNone, "v_exp_f32 | v_cvt_pknorm_i16_f32");
  printf("# -- a third wavefront keeps the matrix pipe busy (32 MFMAs per 192 steps): per step of the VALU streams\n");
  ROW(kMfma, kNone, kNone, "v_mfma_i32_32x32x32_i8 alone (x 6 = cycles per MFMA)");
  ROW(kAdd, kMfma, kNone, "v_add_f32 | MFMA stream");
  ROW(kAdd, kAdd, kMfma, "v_add_f32 | v_add_f32 | MFMA stream");
  ROW(kAdd, kMax3, kMfma, "v_add_f32 | v_max3_i32 | MFMA stream");
  ROW(kExp, kMfma, kNone, "v_exp_f32 | MFMA stream");
  printf("# -- the half-precision softmax tail (conversions to half pairs, dot products of half pairs, the row sum as MFMAs)\n");
  ROW(kCvtPkH, kNone, kNone, "v_cvt_pk_f16_f32 alone");
  ROW(kFmaMix, kNone, kNone, "v_fma_mixlo_f16 alone");
  ROW(kDot2, kNone, kNone, "v_dot2c_f32_f16 alone");
  ROW(kCvtPkH, kAdd, kNone, "v_cvt_pk_f16_f32 | v_add_f32");
  ROW(kCvtPkH, kCvtPkH, kNone, "v_cvt_pk_f16_f32 | v_cvt_pk_f16_f32");
  ROW(kCvtPkH, kMax3, kNone, "v_cvt_pk_f16_f32 | v_max3_i32");
  ROW(kFmaMix, kAdd, kNone, "v_fma_mixlo_f16 | v_add_f32");
  ROW(kFmaMix, kFmaMix, kNone, "v_fma_mixlo_f16 | v_fma_mixlo_f16");
  ROW(kDot2, kAdd, kNone, "v_dot2c_f32_f16 | v_add_f32");
  ROW(kDot2, kDot2, kNone, "v_dot2c_f32_f16 | v_dot2c_f32_f16");
  ROW(kMfmaH, kNone, kNone, "v_mfma_f32_16x16x32_f16 alone (x 4 = cycles per MFMA)");
  ROW(kCvtMfmaH, kNone, kNone, "4 v_cvt_pk_f16_f32 + 1 f16 MFMA, x 32 (x 6 = cycles per group of 5)");
  ROW(kCvtMfmaH, kMfma, kNone, "  the same | int8 MFMA stream (x 6 per group; the int8 stream alone: 32 cycles per MFMA)");
  ROW(kCvtMfmaH, kAdd, kMfma, "  the same | v_add_f32 | int8 MFMA stream");
  ROW(kAdd, kAdd, kNone, "for comparison: the 67 adds of the row sum beside adds (per add)");
  printf("# reading: the SIMD issues two VALU instructions of different wavefronts together when at most one of them is\n"
         "# not plain fp32 add/mul/fma/mov, at most one reads an SGPR, neither is transcendental, and no MFMA is executing.\n");
  return 0;
}
