// LDS access patterns of the attention kernel's operand reads, timed one by one (test tool, gfx950).
//
// The kernel keeps K and V tiles in LDS as [key][d] rows of D bytes and reads them as MFMA operands: K with ds_read_b128
// (lane l: row l % 32, 16-byte chunk l / 32 of the k-step), V with the transposing ds_read_b64_tr_b8 (16-lane groups
// touch keys {0,1,2,3,8,9,10,11} + 4g + 16h).  With plain rows both patterns hit the same banks over and over - the
// "col-major fragment load" conflict of the reference's WMMA kernel (inc/fmha_i8.cuh:155-160) in another guise - and
// the kernel therefore XOR-swizzles the 16-byte chunk index with the row.  This program measures each pattern with and
// without the swizzle against a conflict-free linear read, and each pattern is its own kernel, so that
//
//     rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_INSTS_LDS -- tests/bin/lds_patterns
//
// attributes the bank-conflict cycles to the patterns by name.  Eight wavefronts per CU, each with eight independent
// reads in flight, so that the figure is the throughput of the LDS pipe and not the latency of one read.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                                          \
  do {                                                                                    \
    hipError_t e_ = (x);                                                                  \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
      exit(1);                                                                            \
    }                                                                                     \
  } while (0)

enum Pattern {
  kLinear128,        // ds_read_b128, 16 consecutive bytes per lane: conflict free by construction
  kKPlain128,        // K operand, D = 128, plain rows
  kKSwizzled128,     // K operand, D = 128, chunk ^= (row >> 1) & 7 (what the kernel does)
  kKPlain64,         // K operand, D = 64, plain rows
  kKSwizzled64,      // K operand, D = 64, chunk ^= (row >> 2) & 3
  kLinearTr,         // ds_read_b64_tr_b8, 8 consecutive bytes per lane
  kVPlain128,        // V operand, D = 128, plain rows
  kVSwizzled128,     // V operand, D = 128, chunk ^= (key & 3) | ((key >> 1) & 4)
  kVPlain64,         // V operand, D = 64, plain rows
  kVSwizzled64,      // V operand, D = 64, chunk ^= ((key >> 1) & 1) | ((key >> 2) & 2)
  kKFirstTry128,     // K operand, D = 128, chunk ^= row & 7: rows r and r+8 still collide (two-way conflict)
  kKFirstTry64,      // K operand, D = 64, chunk ^= (row >> 1) & 3: rows r and r+4 still collide
};

// Byte offset of lane l in the j-th of the eight reads a wavefront keeps in flight: the reads of one pass of the real
// kernel over a tile (K: k-steps kk of key tiles t; V: the two halves of key tiles t of output tile 0).
template <int P>
__device__ int lane_offset(int l, int j) {
  const int g = l >> 5, i32 = l & 31;
  if (P == kLinear128) return 16 * l + 1024 * j;
  if (P == kLinearTr) return 8 * l + 512 * j;
  if (P == kKPlain128 || P == kKSwizzled128 || P == kKFirstTry128) {
    const int kk = j & 3, t = j >> 2, sw = P == kKSwizzled128 ? ((i32 >> 1) & 7) : P == kKFirstTry128 ? (i32 & 7) : 0;
    return 4096 * t + i32 * 128 + (((2 * kk + g) ^ sw) << 4);
  }
  if (P == kKPlain64 || P == kKSwizzled64 || P == kKFirstTry64) {
    const int kk = j & 1, t = j >> 1, sw = P == kKSwizzled64 ? ((i32 >> 2) & 3) : P == kKFirstTry64 ? ((i32 >> 1) & 3) : 0;
    return 2048 * t + i32 * 64 + (((2 * kk + g) ^ sw) << 4);
  }
  // V: lane (jin = l % 16, hh = (l / 16) % 2, g) reads 8 bytes of key 4g + {0..3, 8..11}[jin / 2] (+16 for the second
  // half of the operand), chunk hh of output tile 0
  const int jin = l & 15, hh = (l >> 4) & 1, kslot = jin >> 1;
  const int key = 4 * g + (kslot < 4 ? kslot : kslot + 4);
  const int t = j >> 1, half = j & 1;
  if (P == kVPlain128 || P == kVSwizzled128) {
    const int sw = P == kVSwizzled128 ? ((key & 3) | ((key >> 1) & 4)) : 0;
    return (32 * t + 16 * half + key) * 128 + ((hh ^ sw) << 4) + 8 * (jin & 1);
  }
  const int sw = P == kVSwizzled64 ? (((key >> 1) & 1) | ((key >> 2) & 2)) : 0;
  return (32 * t + 16 * half + key) * 64 + ((hh ^ sw) << 4) + 8 * (jin & 1);
}

template <int P>
__global__ __launch_bounds__(512) void lds_pattern(int* out, int iters) {
  __shared__ __attribute__((aligned(16))) int lds[4096];  // one 16 KiB tile, read by all eight wavefronts
  for (int i = threadIdx.x; i < 4096; i += 512) lds[i] = i;
  __syncthreads();
  const unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int*)lds;
  unsigned a[8];
  for (int j = 0; j < 8; ++j) a[j] = base + lane_offset<P>(threadIdx.x & 63, j);
  int sum = 0;
  constexpr bool kTr = P >= kLinearTr && P <= kVSwizzled64;
  for (int it = 0; it < iters; ++it) {
    if (kTr) {
      v2i r[8];
      asm volatile(
          "ds_read_b64_tr_b8 %0, %8\n\tds_read_b64_tr_b8 %1, %9\n\tds_read_b64_tr_b8 %2, %10\n\tds_read_b64_tr_b8 %3, %11\n\t"
          "ds_read_b64_tr_b8 %4, %12\n\tds_read_b64_tr_b8 %5, %13\n\tds_read_b64_tr_b8 %6, %14\n\tds_read_b64_tr_b8 %7, %15\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=v"(r[0]), "=v"(r[1]), "=v"(r[2]), "=v"(r[3]), "=v"(r[4]), "=v"(r[5]), "=v"(r[6]), "=v"(r[7])
          : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7]));
      for (int j = 0; j < 8; ++j) sum += r[j][0] ^ r[j][1];
    } else {
      v4i r[8];
      asm volatile(
          "ds_read_b128 %0, %8\n\tds_read_b128 %1, %9\n\tds_read_b128 %2, %10\n\tds_read_b128 %3, %11\n\t"
          "ds_read_b128 %4, %12\n\tds_read_b128 %5, %13\n\tds_read_b128 %6, %14\n\tds_read_b128 %7, %15\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=v"(r[0]), "=v"(r[1]), "=v"(r[2]), "=v"(r[3]), "=v"(r[4]), "=v"(r[5]), "=v"(r[6]), "=v"(r[7])
          : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(a[4]), "v"(a[5]), "v"(a[6]), "v"(a[7]));
      for (int j = 0; j < 8; ++j) sum += r[j][0] ^ r[j][3];
    }
  }
  if (sum == 0x7fffffff) out[0] = sum;  // (keeps the reads)
}

template <int P>
double run(const char* name, int bytes_per_instr, int* out, int iters) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  hipLaunchKernelGGL(lds_pattern<P>, dim3(256), dim3(512), 0, 0, out, iters);
  CHECK(hipDeviceSynchronize());
  double best = 1e30;
  for (int rep = 0; rep < 3; ++rep) {
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(lds_pattern<P>, dim3(256), dim3(512), 0, 0, out, iters);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    if (ms < best) best = ms;
  }
  // 8 wavefronts x 8 instructions per iteration per CU
  const double ns_per_instr = best * 1e6 / ((double)iters * 64.0);
  printf("%-58s %7.2f ns per wavefront instruction per CU  %7.1f bytes/ns per CU\n", name, ns_per_instr,
         bytes_per_instr / ns_per_instr);
  return ns_per_instr;
}

int main(int argc, char** argv) {
  const int iters = argc > 1 ? atoi(argv[1]) : 4000;
  int* out;
  CHECK(hipMalloc(&out, 256));
  for (int warm = 0; warm < 20; ++warm) hipLaunchKernelGGL(lds_pattern<kLinear128>, dim3(256), dim3(512), 0, 0, out, iters);
  CHECK(hipDeviceSynchronize());
  printf("# LDS operand-read patterns, 256 workgroups x 8 wavefronts, 8 reads in flight per wavefront\n");
  const double lin = run<kLinear128>("ds_read_b128 linear (conflict free)", 1024, out, iters);
  const double kp = run<kKPlain128>("ds_read_b128 K operand d=128, plain [key][d] rows", 1024, out, iters);
  const double kf = run<kKFirstTry128>("ds_read_b128 K operand d=128, chunk ^ (row & 7)  [first try]", 1024, out, iters);
  const double ks = run<kKSwizzled128>("ds_read_b128 K operand d=128, chunk ^ ((row >> 1) & 7)", 1024, out, iters);
  const double kp64 = run<kKPlain64>("ds_read_b128 K operand d=64, plain rows", 1024, out, iters);
  const double kf64 = run<kKFirstTry64>("ds_read_b128 K operand d=64, chunk ^ ((row >> 1) & 3)  [first try]", 1024, out, iters);
  const double ks64 = run<kKSwizzled64>("ds_read_b128 K operand d=64, chunk ^ ((row >> 2) & 3)", 1024, out, iters);
  const double lt = run<kLinearTr>("ds_read_b64_tr_b8 linear", 512, out, iters);
  const double vp = run<kVPlain128>("ds_read_b64_tr_b8 V operand d=128, plain rows", 512, out, iters);
  const double vs = run<kVSwizzled128>("ds_read_b64_tr_b8 V operand d=128, swizzled", 512, out, iters);
  const double vp64 = run<kVPlain64>("ds_read_b64_tr_b8 V operand d=64, plain rows", 512, out, iters);
  const double vs64 = run<kVSwizzled64>("ds_read_b64_tr_b8 V operand d=64, swizzled", 512, out, iters);
  printf("# K d=128: plain / swizzled = %.2fx, swizzled / linear = %.2fx;  V d=128: plain / swizzled = %.2fx, swizzled / linear = %.2fx\n",
         kp / ks, ks / lin, vp / vs, vs / lt);
  printf("# K d=64:  plain / swizzled = %.2fx;  V d=64: plain / swizzled = %.2fx\n", kp64 / ks64, vp64 / vs64);
  printf("# K, first-try swizzle / final swizzle: d=128 %.2fx, d=64 %.2fx\n", kf / ks, kf64 / ks64);
  return 0;
}
