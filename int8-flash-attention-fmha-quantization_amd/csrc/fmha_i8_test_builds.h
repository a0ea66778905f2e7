// Test builds of the attention kernel (tests/Makefile, target `variants`; never the shipped library).
//
// They exist so that every claim about where the time goes can be re-measured: each one removes or changes ONE thing
// and is timed and counted against the shipped kernel (tests/variant_timing.py).  The knock-outs produce garbage results
// on purpose.  Everything here is decided at compile time: in the shipped build every flag below is false, the kernel's
// `if constexpr (test_build::...)` branches are discarded and the staged-load macro at the end is empty.
//
//   FMHA_KO_SOFTMAX      the block softmax is not computed (P, block maximum and row sum are left undefined)
//   FMHA_KO_MFMA         GEMM 2 + merge and GEMM 1 + row maximum are not computed (with FMHA_KO_SOFTMAX: the key loop
//                        is tile loads, waits and barriers only)
//   FMHA_KO_SCALE_RUN, FMHA_KO_EXP_RUN, FMHA_KO_SUM_RUN   one of the three dense runs of the steady-state softmax is
//                        left out: the 64 scale fmas (and conversions), the 64 exponentials, the 64 + 4 row-sum adds
//   FMHA_KO_LDS_READS    the MFMA operands are undefined registers instead of LDS reads
//   FMHA_KO_TILE_LOADS   no K/V tile is fetched after the prologue
//   FMHA_NO_SWIZZLE      K and V tiles lie in LDS as plain [key][d] rows (results unchanged, bank conflicts are not)
//   FMHA_OLD_K_SWIZZLE   the K swizzle this kernel had first, which leaves a two-way conflict on every K operand read
//   FMHA_TRACE_TICKS     every wavefront records the shader-clock time of each barrier arrival and departure
//   FMHA_VGPR_STAGED_LOADS  the "before" of the direct-to-LDS tile loads: in the steady-state loop at d = 128 a K/V tile
//                        goes HBM -> registers (global_load_dwordx4) and, one key block later, registers -> LDS
//                        (ds_write_b128), the way a kernel without LDS-DMA has to do it; same bytes in the same places
//   FMHA_TWO_BARRIERS    the "before" of the one-barrier schedule: a second workgroup barrier per key block, between the
//                        two phases (results unchanged)
//   FMHA_MFMA_ROWSUM     the row sum of the steady-state softmax on the matrix pipe: the exponentials rounded to half
//                        precision two at a time (v_cvt_pk_f16_f32) and summed by v_mfma_f32_16x16x32_f16 against an
//                        operand of ones, 32 conversions and 8 MFMAs in place of 67 additions (results within the usual
//                        gate of the shipped kernel's, not bit-identical; measured slower)
//   FMHA_CHECK_BOUNDS    every global access of the kernel is first checked against the tensor - for K and V the head -
//                        it belongs to; an access that would leave it is counted in g_fmha_oob_count and redirected to
//                        the first byte, so that the run ends normally and the test can read the count.  An
//                        out-of-bounds READ changes no result and, inside a caching allocator's pool, raises no fault:
//                        nothing else shows it.
//   FMHA_LOOP_PAD_A=n    n s_nops between the 64-byte boundary in front of the steady-state loop of wavefronts 0..3 and
//                        the loop (the kernel's own choice otherwise): for re-measuring what the placement costs
#pragma once

namespace fmha_i8_gfx950 {
namespace test_build {

#ifdef FMHA_KO_SOFTMAX
constexpr bool kNoSoftmax = true;
#else
constexpr bool kNoSoftmax = false;
#endif
#ifdef FMHA_KO_MFMA
constexpr bool kNoMfma = true;
#else
constexpr bool kNoMfma = false;
#endif
#ifdef FMHA_KO_SCALE_RUN
constexpr bool kNoScaleRun = true;
#else
constexpr bool kNoScaleRun = false;
#endif
#ifdef FMHA_KO_EXP_RUN
constexpr bool kNoExpRun = true;
#else
constexpr bool kNoExpRun = false;
#endif
#ifdef FMHA_KO_SUM_RUN
constexpr bool kNoSumRun = true;
#else
constexpr bool kNoSumRun = false;
#endif
#ifdef FMHA_KO_LDS_READS
constexpr bool kNoLdsReads = true;
#else
constexpr bool kNoLdsReads = false;
#endif
#ifdef FMHA_KO_TILE_LOADS
constexpr bool kNoTileLoads = true;
#else
constexpr bool kNoTileLoads = false;
#endif
#ifdef FMHA_NO_SWIZZLE
constexpr bool kNoSwizzle = true;
#else
constexpr bool kNoSwizzle = false;
#endif
#ifdef FMHA_OLD_K_SWIZZLE
constexpr bool kOldKSwizzle = true;
#else
constexpr bool kOldKSwizzle = false;
#endif
#ifdef FMHA_TWO_BARRIERS
constexpr bool kTwoBarriers = true;
#else
constexpr bool kTwoBarriers = false;
#endif
#ifdef FMHA_VGPR_STAGED_LOADS
constexpr bool kStagedLoads = true;
#else
constexpr bool kStagedLoads = false;
#endif
#ifdef FMHA_MFMA_ROWSUM
constexpr bool kMfmaRowSum = true;
#else
constexpr bool kMfmaRowSum = false;
#endif
#ifdef FMHA_TRACE_TICKS
constexpr bool kTraceTicks = true;
#else
constexpr bool kTraceTicks = false;
#endif
#ifdef FMHA_LOOP_PAD_A
constexpr int kLoopPadA = FMHA_LOOP_PAD_A;
#else
constexpr int kLoopPadA = -1;  // the kernel's own choice
#endif

// What a knocked-out producer leaves behind: a register (or a vector of them) whose content is undefined, at no cost.
template <class T>
__device__ __forceinline__ void undefined(T& x) {
  asm volatile("" : "=v"(x));
}
// ... and what a knocked-out consumer does with its inputs: it names them, so that their producers stay.
template <class T>
__device__ __forceinline__ void consume(const T& x) {
  asm volatile("" ::"v"(x));
}

}  // namespace test_build

#ifdef FMHA_CHECK_BOUNDS
__device__ int g_fmha_oob_count;
__device__ __forceinline__ bool fmha_in_bounds(bool ok) {
  if (!ok) atomicAdd(&g_fmha_oob_count, 1);
  return ok;
}
#else
__device__ __forceinline__ constexpr bool fmha_in_bounds(bool) { return true; }
#endif

#ifdef FMHA_TRACE_TICKS
// [workgroup][wavefront][64]: lane n < 62 of one register holds the n-th time stamp (s_memtime, shader clock), lanes 62
// and 63 the 100 MHz counter at the start and the end of the wavefront; written out when the wavefront ends.
constexpr int kTraceWorkgroups = 4096;
__device__ unsigned g_fmha_trace[kTraceWorkgroups * 8 * 64];
namespace test_build {
__device__ __forceinline__ void write_trace(unsigned workgroup, int wave, int lane, unsigned stamps) {
  if (workgroup < kTraceWorkgroups) g_fmha_trace[(workgroup * 8 + wave) * 64 + lane] = stamps;
}
}  // namespace test_build
#else
namespace test_build {
__device__ __forceinline__ void write_trace(unsigned, int, int, unsigned) {}
}  // namespace test_build
#endif

}  // namespace fmha_i8_gfx950

// The register-staged tile path of FMHA_VGPR_STAGED_LOADS, expanded inside the kernel where its key loop is set up (it
// uses the kernel's own names: the tile geometry, the LDS ring, the per-lane load offsets).  One pair of tiles
// (K(i+3), V(i+2)) is on its way through this wavefront's registers: loaded at the issue point of key block i, written
// to LDS at the issue point of key block i+1 - still a whole key block before the barrier that publishes it.  Only where
// the tiles would otherwise be requested in front of the MFMA phase (d = 128).  LDS writes are not waited for by the
// hand-written barrier, hence staged_writes_done().
#ifdef FMHA_VGPR_STAGED_LOADS
#define FMHA_STAGED_LOAD_LAMBDAS                                                                                         \
  constexpr bool kStaged = kOneBarrier && !kLoadsInMfmaPhase && !RAGGED;                                                  \
  v4i staged[2][kRegionsPerWave];                                                                                         \
  int staged_kb[2] = {0, 0};                                                                                              \
  bool have_staged = false;                                                                                               \
  auto staged_write = [&]() {                                                                                             \
    if (!have_staged) return;                                                                                             \
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                                      \
    _Pragma("unroll") for (int which = 0; which < 2; ++which)                                                             \
      _Pragma("unroll") for (int it = 0; it < kRegionsPerWave; ++it) {                                                    \
        asm volatile("" : "+v"(staged[which][it]));                                                                       \
        const int region = (it * kWaves + wave) % kRegions;                                                               \
        *reinterpret_cast<v4i*>(&lds[staged_kb[which] & (kStages - 1)][which][region * 1024 + 16 * lane]) =               \
            staged[which][it];                                                                                            \
      }                                                                                                                   \
    have_staged = false;                                                                                                  \
  };                                                                                                                      \
  auto staged_step = [&](int i) {                                                                                         \
    staged_write();                                                                                                       \
    staged_kb[0] = min(i + 3, last);                                                                                      \
    staged_kb[1] = min(i + 2, last);                                                                                      \
    _Pragma("unroll") for (int which = 0; which < 2; ++which)                                                             \
      _Pragma("unroll") for (int it = 0; it < kRegionsPerWave; ++it) {                                                    \
        const int8_t* gp = (which ? vg : kg) + (long)staged_kb[which] * kTileBytes;                                       \
        const int region = (it * kWaves + wave) % kRegions;                                                               \
        const int src = (which ? ld_goff_v : ld_goff_k) + region * 1024;                                                  \
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(staged[which][it]) : "v"(src), "s"(gp) : "memory");          \
      }                                                                                                                   \
    have_staged = true;                                                                                                   \
  };                                                                                                                      \
  auto staged_writes_done = [&]() { if (kStaged) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };
#else
#define FMHA_STAGED_LOAD_LAMBDAS        \
  constexpr bool kStaged = false;       \
  auto staged_write = [&]() {};         \
  auto staged_step = [&](int) {};       \
  auto staged_writes_done = [&]() {};
#endif
