// INT8 fused multi-head flash attention for gfx950 (MI355X, CDNA4).  One kernel, templated on head_dim.
//
// What it computes is what the reference's FMHAInferKernel computes (inc/fmha_i8.cuh:43-334): per (batch, head),
// S = Q.K^T in int32, dequantised by 1/sqrt(d) * q_amax*k_amax/127^2, softmax over blocks of 128 keys against the
// BLOCK-LOCAL row maximum, P requantised to int8 in [-128,0] (scale -128, round-half-even), O~ = P.V in int32,
// online (m, l, O) merge across key blocks, and O requantised to int8 with v_amax/(128*o_amax), clamp +-127.
//
// How it computes it is designed for CDNA4, not taken from the reference:
//   * grid over (query block of 256 rows) x head x batch, XCD-aware so that the query blocks of one head share an L2;
//     one workgroup of 8 wavefronts per CU, each wavefront owns 32 query rows, two wavefronts per SIMD;
//   * both GEMMs run on v_mfma_i32_32x32x32_i8 in the TRANSPOSED formulation S^T = K.Q^T and O^T = V^T.P^T: each
//     lane then owns one query column, so the row max / row sum are in-register reductions plus one exchange with
//     lane^32, and the quantised P^T tile leaves the accumulator already in the B-operand register layout;
//   * K and V tiles of 128 keys go HBM -> LDS directly (global_load_lds_dwordx4, no VGPR staging, no ds_write) into
//     a ring of four stages, fetched three key blocks ahead, as [key][d] with the 16-byte chunk index XOR-swizzled by
//     the row (the swizzle is applied to the global address each lane fetches), so that the 128-bit operand reads of
//     K and the transposing reads of V (ds_read_b64_tr_b8) are bank-conflict free; Q goes once per workgroup straight
//     into MFMA operand registers;
//   * the kernel is bound by the instruction issue of the SIMD (a VALU instruction takes 4.3 to 4.7 cycles of it, an
//     exponential 8.5, an MFMA 10 to 12; two wavefronts rarely issue together), so the two wavefronts that share a SIMD
//     run in ANTI-PHASE: every key block is an MFMA phase - GEMM 2 and merge of the previous block, then GEMM 1 of this
//     one, with the merge and the row maximum issued in the shadow of the MFMAs - and a VALU phase, the softmax;
//     wavefronts 4..7 run one phase behind wavefronts 0..3, and the wavefront in its MFMA phase runs at raised priority,
//     so that the MFMA pipe never waits for an issue slot.  One workgroup barrier per key block publishes the tiles;
//   * the softmax is written for instruction count and issue order: exp in the base-2 domain with every scale folded
//     into one fma, v_max3 on the raw accumulators for the row maximum, P converted two at a time by
//     v_cvt_pknorm_i16_f32 and packed by v_perm_b32, the steady-state loops running the scale fmas, the exponentials
//     and the sums as three dense runs with the P packing at the head of the MFMA phase, the general loop (the last
//     block) with every exponential followed by instructions that do not need the transcendental unit, the
//     int32 accumulators of both GEMMs started at the bit pattern of a float (an MFMA inline
//     constant) so that they can be read as floats without a convert, the running O only rescaled when a row maximum
//     jumps by more than 2^kLazyLog2, and O normalised once, in the epilogue.
//   * masked keys (nonzero mask byte) cost the softmax nothing: GEMM 1 of a block that has some STARTS their accumulators
//     at a value that loses every maximum and whose exponential is exactly 0; blocks whose keys are all masked are
//     skipped.  The mask of a batch entry is classified once per workgroup, by wavefronts 0..3, in the prologue;
//   * a second set of instantiations (FULLP) keeps P on all 255 steps of a byte - planned by the reference, README.md:15,186
//     - by computing with P - 128 and starting the GEMM 2 accumulators at 128 times the column sums of the V tile.
#include <hip/hip_runtime.h>
#include <stdint.h>

// No floating-point contraction by the compiler: every fused multiply-add in this file is written out
// (__builtin_fmaf), so the bits of the result do not depend on which products the optimiser decides to fuse.
#pragma clang fp contract(off)

namespace fmha_i8_gfx950 {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBlockQ = 256;   // query rows per workgroup
constexpr int kBlockK = 128;   // keys per softmax block (the reference's BASE_SEQ_LEN, src/fmha_i8.cu:61-95) ...
constexpr int kBlockKSmall = 64;  // ... and for its sequence lengths that are odd multiples of 64 (src/fmha_i8.cu:41-60)
constexpr int kThreads = 512;  // 8 wavefronts: 0..3 and 4..7 run the key-block phases one phase apart
constexpr int kStages = 4;     // K/V tiles resident in LDS per kind: a tile is fetched several phases before its first use
constexpr int kXcds = 8;
constexpr int kMaxKeyBlocks = 1024;      // seq_len <= 65536, also in blocks of 64 keys
constexpr float kMagic = 12582912.0f;    // 1.5 * 2^23: kMagic + y holds rne(y) in its low mantissa bits (output rounding)
// Both GEMMs start their int32 accumulators at the bit pattern of the float 1/(2 pi), held in sixteen registers that
// the first MFMA of every chain names as its C operand.  That float sits 2292099 ulps above 2^-3 and 6096509 below 2^-2,
// more than any int8 dot product of 128 terms can reach (|x| <= 2^21), so kBaseBits + x read as a float is exactly
// kBase + x * 2^-26: the integer result is available to float arithmetic without a convert.
constexpr int kBaseBits = 0x3E22F983;
constexpr float kBase = __builtin_bit_cast(float, kBaseBits);
constexpr float kBaseScale = 67108864.0f;  // 2^26: float units per integer unit, inverted
// The accumulators of GEMM 1 at head_dim 64 start lower in the same binade: 0x110000 = 1114112 ulps above 2^-3, more than
// the 127*127*64 = 1032256 a dot product of 64 terms can reach.  The exponent offset of the biased path is rounded at the
// magnitude (start value in ulps + S) * c2, and the lower start extends the range of score scales that path can serve by
// a half (N(0,1) inputs at head_dim 64 fall inside it); GEMM 2 sums 128 keys whatever the head_dim and keeps kBaseBits.
constexpr int kBaseBitsScores64 = 0x3E110000;
template <int D>
constexpr int score_base_bits() { return D == 64 ? kBaseBitsScores64 : kBaseBits; }
template <int D>
constexpr float score_base_ulps() { return (float)(score_base_bits<D>() - 0x3E000000) + 8388608.0f; }  // the start value / 2^-26
template <int D>
constexpr float score_range_ulps() { return D == 64 ? 1048576.0f : 4194304.0f; }  // bound on |S| used by the host
constexpr float kBiasOffsetLimit = 4096.0f;  // see the launch code: bound on the exponent offset of the biased path
constexpr float kLog2Pscale = -7.99995597f;  // log2(128 / 32767): exp2(x + kLog2Pscale) = 128 p / 32767
constexpr float kLazyLog2 = 10.0f;       // the running O is rescaled only when a row maximum grows by more than this
// Full-range P (the FULLP variant below): P = rne(255 p) in [0, 255], so |sum of P v| over 128 keys can reach
// 255 * 127 * 128 = 4145280.  Its GEMM 2 accumulators start at the float 0.1875, which sits exactly 2^22 = 4194304
// ulps from either end of its binade.
constexpr float kLog2PscaleFull = -7.00560236f;  // log2(255 / 32767)
constexpr int kBaseBitsFull = 0x3E400000;
constexpr float kBaseFull = __builtin_bit_cast(float, kBaseBitsFull);

}  // namespace fmha_i8_gfx950

// Test builds (knock-outs, "before" layouts and schedules, time stamps, bounds checks): compile-time flags, all false
// in the shipped library, and the few helpers they need.  `fmha_in_bounds` comes from there too: it is the constant
// `true` unless the build checks every global access.
#include "fmha_i8_test_builds.h"

namespace fmha_i8_gfx950 {

struct KernelArgs {
  const int8_t* q;
  const int8_t* k;
  const int8_t* v;
  const int8_t* mask;
  int8_t* o;
  int seq_q;        // query (and output) rows per head: any positive count
  int seq_kv;       // key/value rows per head and mask bytes per batch entry: any positive count; keys from there to
                    // the next multiple of BK do not exist and count as masked
  int head_num;
  int q_blocks;     // ceil(seq_q / kBlockQ)
  int total_wgs;    // batch * head_num * q_blocks
  float c2;         // log2(e) * (1/sqrt(d)) * q_amax*k_amax/127^2 : int32 S -> base-2 exponent
  float floor2;     // log2(e) * -1e6 : the reference's initial block maximum (inc/fmha_i8.cuh:116)
  float out_scale;  // v_amax / (o_amax * 128)   (inc/fmha_i8.cuh:318)
};

// 16-byte-chunk swizzles.  K is read 32 consecutive rows at a time (ds_read_b128); V is read by ds_read_b64_tr_b8
// whose 16-lane groups touch keys {0,1,2,3,8,9,10,11} (+4, +16, +20) of a 32-key slab.
template <int D>
__device__ __forceinline__ int k_swizzle(int row) {
  if constexpr (test_build::kNoSwizzle) return 0;
  // (the swizzle this kernel had first: rows r and r+8 / r+4 collide, a two-way conflict)
  if constexpr (test_build::kOldKSwizzle) return D == 128 ? (row & 7) : ((row >> 1) & 3);
  // Sixteen lanes are served per cycle: rows r .. r+15 of one 16-byte chunk column.  A row is D bytes, the banks repeat
  // every 256 bytes, so rows 256/D apart start in the same bank: those rows must get different chunks.
  return D == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}
template <int D>
__device__ __forceinline__ int v_swizzle(int key) {
  if constexpr (test_build::kNoSwizzle) return 0;
  return D == 128 ? ((key & 3) | ((key >> 1) & 4)) : (((key >> 1) & 1) | ((key >> 2) & 2));
}

// P packing: four floats y_i in [-1, 1] -> four int8 bytes rne(32767 * y_i).  v_cvt_pknorm_i16_f32 converts two at a
// time (round to nearest; exact .5 ties toward zero, which real softmax values do not hit), v_perm_b32 keeps the low
// byte of each 16-bit result.
typedef short v2s __attribute__((ext_vector_type(2)));
constexpr float kSnorm = 32767.0f;

// Lanes l and l^32 hold the two halves of one query column: v_permlane32_swap hands each lane both halves.
__device__ __forceinline__ float half_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_int(x), __float_as_int(x), false, false);
  return fmaxf(__int_as_float(r[0]), __int_as_float(r[1]));
}
__device__ __forceinline__ int half_max(int x) {
  const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  return max((int)r[0], (int)r[1]);
}
__device__ __forceinline__ float half_sum(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_int(x), __float_as_int(x), false, false);
  return __int_as_float(r[0]) + __int_as_float(r[1]);
}

// BIAS: the S accumulators start at the bit pattern of a float (kBaseBits; kBaseBitsScores64 at head_dim 64) and are read
// as floats (no int->float convert).  Exact only while (start value * 2^26 + |S|) * c2 stays small enough for the float
// grid; the host selects it from c2.
// FASTACC: the running O absorbs the kBase offset of the GEMM 2 accumulators (one fma per element and key block
// instead of subtract + fma) and the offset is taken out once, in the epilogue.  O then lives near kBase * sum(take)
// and each merge rounds at that magnitude; the host enables it only where that rounding is far below one output LSB.
// RAGGED: seq_kv is not a multiple of BK.  Everything that serves the partly filled last block is compiled in only
// then: in the key loop it costs some fifty scalar instructions per block, which the other lengths do not pay.
// FULLP: P keeps all 255 steps of a byte, P = rne(255 p) - what the reference plans as "uint8 x int8" (README.md:15,186)
// and has no code for.  The matrix unit multiplies signed bytes only, so GEMM 2 runs on P - 128 (the byte with its top
// bit flipped) and the missing 128 * sum_j v[j][c] per key block and output column goes in as the START VALUE of the
// accumulators: wavefronts 4..7 sum the columns of every V tile one phase before its GEMM 2 (v_dot4 on the transposed
// operand reads), leave kBaseBitsFull + 128 * sum in LDS, and every wavefront reads its C operand from there.
template <int D, int BK, bool BIAS, bool FASTACC, bool RAGGED, bool FULLP>
__global__ __launch_bounds__(kThreads, 2) void fmha_i8_fwd_kernel(const KernelArgs args) {
  constexpr int kChunks = D / 16;                     // 16-byte chunks per row
  constexpr int kTileBytes = BK * D;                  // one K or V tile
  constexpr int kWaves = kThreads / 64;
  constexpr int kRegions = kTileBytes / 1024;         // 1 KiB (64 lanes x 16 B) direct-to-LDS loads per tile
  constexpr int kRegionsPerWave = (kRegions + kWaves - 1) / kWaves;  // ... and per wavefront (a tile of fewer regions
                                                      // than wavefronts is loaded twice: all wavefronts count alike)
  constexpr int kRowsPerRegion = 1024 / D;
  constexpr int kDSteps = D / 32;                     // MFMA k-steps of GEMM 1, and 32-row output tiles of GEMM 2
  constexpr int kKeyTiles = BK / 32;

  __shared__ __attribute__((aligned(1024))) int8_t lds[kStages][2][kTileBytes];  // [stage][K|V][tile]; tile j -> stage j % kStages
  __shared__ unsigned char lds_class[kMaxKeyBlocks];  // per key block: bit0 = some key masked, bit1 = all keys masked
  __shared__ unsigned lds_mask[kMaxKeyBlocks * kBlockKSmall / 32];  // bit j%32 of word j/32: key j of this batch entry is masked
  __shared__ __attribute__((aligned(16))) int lds_colsum[FULLP ? 2 * D : 4];  // FULLP: [key block & 1][output column]
  __shared__ __attribute__((aligned(16))) int lds_scan[8];  // per classifying wavefront: last block with an unmasked key, first block with a masked one

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;   // which 16-byte k-slot group of the 32x32x32 MFMA this lane feeds
  const int i32 = lane & 31; // MFMA row/column index of this lane

  // XCD-aware placement: hardware hands consecutive workgroup ids to consecutive XCDs; give every XCD a contiguous
  // range of (head, query block) so that the query blocks of a head hit the same L2.
  int wg;
  {
    const int L = blockIdx.x, per = args.total_wgs / kXcds, rem = args.total_wgs % kXcds, x = L % kXcds;
    wg = x * per + (x < rem ? x : rem) + L / kXcds;
  }
  const int bh = wg / args.q_blocks;
  const int qb = wg - bh * args.q_blocks;
  const int b = bh / args.head_num;
  const int S = args.seq_kv;
  const int Sq = args.seq_q;
  const long head_off = (long)bh * S * D;    // of K and V
  const long q_head_off = (long)bh * Sq * D; // of Q and O
  const int8_t* __restrict__ kg = args.k + head_off;
  const int8_t* __restrict__ vg = args.v + head_off;
  const int8_t* __restrict__ mg = args.mask + (long)b * S;
  const int n_blocks = (S + BK - 1) / BK;
  const int S_pad = n_blocks * BK;
  // A last key block that is only partly there: its tile loads must not run past the end of K and V.  When it is
  // not the only block its tiles are fetched from BK rows earlier than their place, so that they END with the last key
  // (a change of the wave-uniform base address and nothing else): LDS row r then holds key S - BK + r, the first
  // BK - tail_rows rows repeat keys of the block before and are masked like the padding they stand for.  A sequence
  // shorter than one block is fetched in the prologue with the rows past its end redirected to its last key.
  const int tail_rows = S - (n_blocks - 1) * BK;
  const int tail_kb = (RAGGED && n_blocks > 1) ? n_blocks - 1 : -1;  // the block with the shifted window
  const bool short_seq = RAGGED && S < BK;

  // The prologue puts every cold miss in flight before it waits for any of them: the mask bytes, the first two K/V
  // tiles (tile 1 on speculation: it exists whenever seq_kv >= 256, whether or not its keys are masked) and the Q rows.
  // (Every lambda of this kernel that touches the register-resident state - accumulators, running O, Q - is marked
  // always_inline: one that the compiler decided to call instead would force what it captures by reference into
  // scratch memory.)
  // ---- per-lane addressing -----------------------------------------------------------------------------------------
  // direct-to-LDS loads: lane l of a 1 KiB region lands at byte 16*l of the region, so the lane FETCHES the chunk that
  // the swizzle assigns to that slot.
  int ld_goff_k, ld_goff_v;
  const int ld_row_in = lane / kChunks;
  {
    const int row_in = ld_row_in, p = lane % kChunks;
    // A 1 KiB region is 8 rows at D = 128 and this wavefront's regions all have the parity of its index: that is the
    // one row bit beyond row_in that the swizzles look at.
    const int vrow = (D == 128) ? (row_in | ((wave & 1) << 3)) : row_in;
    ld_goff_k = row_in * D + ((p ^ k_swizzle<D>(vrow)) << 4);
    ld_goff_v = row_in * D + ((p ^ v_swizzle<D>(vrow)) << 4);
  }
  int k_read_off[kDSteps];  // + 32*t*D per key tile
#pragma unroll
  for (int kk = 0; kk < kDSteps; ++kk)
    k_read_off[kk] = i32 * D + (((2 * kk + g) ^ k_swizzle<D>(i32)) << 4);
  int v_read_off[kDSteps];  // + 32*t*D per key tile, + 16*D for the second half of the operand
  int colsum_tile, colsum_read_off;
  {
    const int jin = lane & 15, hh = (lane >> 4) & 1;
    const int kslot = jin >> 1;
    const int key_lane = 4 * g + (kslot < 4 ? kslot : kslot + 4);
#pragma unroll
    for (int u = 0; u < kDSteps; ++u)
      v_read_off[u] = key_lane * D + (((2 * u + hh) ^ v_swizzle<D>(key_lane)) << 4) + 8 * (jin & 1);
    // FULLP: wavefront 4 + u sums the columns of output tile u (the same operand reads, a run-time tile index)
    colsum_tile = wave - 4;
    colsum_read_off = key_lane * D + (((2 * (colsum_tile & (kDSteps - 1)) + hh) ^ v_swizzle<D>(key_lane)) << 4) + 8 * (jin & 1);
  }

  // HBM -> LDS without passing through registers.  Written as inline assembly on purpose: the compiler treats an
  // LDS-DMA builtin as a store that may alias every later LDS read and would wait for tiles that are still in flight
  // before the first operand read of the current one.  Completion is tracked by hand with s_waitcnt vmcnt(n) in front
  // of the barrier that publishes a tile.  M0 carries the LDS destination of lane 0; lane l lands 16*l bytes further.
  // (M0 cannot be named as a clobber: the compiler reserves it and rejects it on a clobber list.  Every statement here
  // that needs M0 sets it itself, in the same statement, so none depends on what another one left there.)
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int8_t*)&lds[0][0][0];
  // Tile 0 of a sequence shorter than one block - the only tile there is, fetched in the prologue and again at every
  // later issue point: rows past the last key fetch the last key instead (same chunk: the swizzle belongs to the LDS
  // row); what lands there is never attended to, those keys are masked.  Fetching the whole tile would read up to
  // BK - S rows past the end of K and V.
  auto issue_short_region = [&](const int8_t* gbase, int which, int goff, int region) __attribute__((always_inline)) {
    const unsigned dst = lds_base + (unsigned)(which * kTileBytes + region * 1024);
    const int row = region * kRowsPerRegion + ld_row_in;
    int src = goff + region * 1024 - (row >= S ? (row - (S - 1)) * D : 0);
    if (!fmha_in_bounds(src >= 0 && src + 16 <= S * D)) src = 0;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(dst), "v"(src), "s"(gbase) : "memory");
  };
  bool prologue_done = false;  // (the test build without tile loads still fetches the tiles of the prologue)
  // (steady: called from a steady-state loop, which a sequence of less than one key block never enters - said at compile
  // time, so that those loops carry no branch for it)
  auto issue_region = [&](const int8_t* gbase, int kb, int which, int goff, int it, bool steady = false) __attribute__((always_inline)) {  // which: 0 = K, 1 = V
    if (test_build::kNoTileLoads && prologue_done) return;
    const int region = (it * kWaves + wave) % kRegions;
    if (RAGGED && !steady && short_seq) {
      issue_short_region(gbase, which, goff, region);
      return;
    }
    const int8_t* gp = gbase + (long)kb * kTileBytes;  // wave-uniform base (SGPR pair)
    if (RAGGED && kb == tail_kb) gp = gbase + (long)(S - BK) * D;
    const unsigned dst = lds_base + (unsigned)(((kb & (kStages - 1)) * 2 + which) * kTileBytes + region * 1024);
    int src = goff + region * 1024;
    {
      const long rel = (long)(gp - gbase) + src;  // offset inside the head
      if (!fmha_in_bounds(rel >= 0 && rel + 16 <= (long)S * D)) src = (int)(gbase - gp);
    }
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(dst), "v"(src), "s"(gp) : "memory");
  };
  // Region `region` of tile 0 (the prologue, where the tiles are split between the wavefronts differently)
  auto issue_region0_at = [&](const int8_t* gbase, int which, int goff, int region) __attribute__((always_inline)) {
    if (RAGGED && short_seq) {
      issue_short_region(gbase, which, goff, region);
      return;
    }
    const int8_t* gp = gbase;
    if (RAGGED && tail_kb == 0) gp = gbase + (long)(S - BK) * D;
    const unsigned dst = lds_base + (unsigned)(which * kTileBytes + region * 1024);
    int src = goff + region * 1024;
    {
      const long rel = (long)(gp - gbase) + src;  // offset inside the head
      if (!fmha_in_bounds(rel >= 0 && rel + 16 <= (long)S * D)) src = (int)(gbase - gp);
    }
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(dst), "v"(src), "s"(gp) : "memory");
  };
  // Tile 0 in the prologue: K0 is fetched by wavefronts 0..3 alone and V0 by wavefronts 4..7 alone (regions
  // (wave & 3) + 4 it: the same parity as the wavefront's regions in the key loop, which the swizzled offsets assume),
  // so that the first barrier, which publishes K0, does not wait for the wavefronts that start last.
  constexpr int kPrologueRegions = (kRegions + 3) / 4;
  auto issue_tile0_by_half = [&](const int8_t* gbase, int which, int goff) __attribute__((always_inline)) {
#pragma unroll
    for (int it = 0; it < kPrologueRegions; ++it) issue_region0_at(gbase, which, goff, (4 * it + (wave & 3)) % kRegions);
  };
  auto issue_tile = [&](const int8_t* gbase, int kb, int which, int goff) __attribute__((always_inline)) {
#pragma unroll
    for (int it = 0; it < kRegionsPerWave; ++it) issue_region(gbase, kb, which, goff, it);
  };
  auto issue_k = [&](int kb) __attribute__((always_inline)) { issue_tile(kg, kb, 0, ld_goff_k); };
  auto issue_v = [&](int kb) __attribute__((always_inline)) { issue_tile(vg, kb, 1, ld_goff_v); };
  // Memory reads return in issue order: waiting until at most `tiles` tiles of this wavefront's loads are outstanding
  // retires every tile older than the newest `tiles` ones.
  auto wait_all_but = [&](int tiles) {
    if (tiles >= 4) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(4 * kRegionsPerWave) : "memory");
    else if (tiles == 3) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(3 * kRegionsPerWave) : "memory");
    else if (tiles == 2) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * kRegionsPerWave) : "memory");
    else if (tiles == 1) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kRegionsPerWave) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  auto wait_all = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
  // A VALU instruction with a 64-bit encoding issues in 4.7 cycles from an 8-byte-aligned address and in 5.4 to 5.7 from
  // an address that is 4 mod 8 (one instruction per fetch of an aligned pair of dwords); the compiler aligns nothing
  // inside a function.  The d = 64 kernel is sensitive to where the MFMAs of GEMM 1 and the row-maximum instructions
  // behind them fall (+12 % when they straddle), so it pins those, the scale fmas and the P packing to aligned
  // addresses; the d = 128 kernel measures the same either way (+-0.3 %) in its loop without masked keys and is left
  // alone there (pinning everything costs it 0.4 %).  Its loop for blocks WITH masked keys is sensitive (up to 9 % between
  // two placements, B1 H4 S8192 with a scattered mask), so that loop pins the same groups, and GEMM 1 with start values
  // pins each tile's run of v_cndmask and its MFMAs at either head size: 1.5 to 3 % faster and 3 % left between
  // placements.
  auto align8 = [&](bool also_at_128 = false) { if (D == 64 || also_at_128) asm volatile(".p2align 3" ::: "memory"); };
  // The steady-state loops start at a fixed distance from a 64-byte boundary, so that what is measured for them does
  // not change with the code in front of them: at d = 64 the loop of wavefronts 0..3 runs 12 % slower when it starts
  // 4 bytes further on or back (B16 H16 S2048: 226 against 254 us; every even distance measures the same, every odd
  // one too; the loop of wavefronts 4..7 measures the same either way, and so do both loops at d = 128).  What flips
  // with those 4 bytes is whether the eight v_max3_i32 at the top of the loop - the first readers of the last MFMA of
  // GEMM 1 - start at 8-byte-aligned addresses (fast) or straddle two (slow).  The right distance is found by timing
  // (the test builds loop_pad_a0 and loop_pad_a1, -DFMHA_LOOP_PAD_A=0 against 1) whenever the code between the boundary
  // and the loop changes; tests/test_gpu_variant_builds.py holds the shipped library to the faster of the two.
  auto align_loop = [&]() { asm volatile(".p2align 6" ::: "memory"); };
  // s_nops between the boundary and the loop of wavefronts 0..3 (see above): the 255-step variant has other code
  // between the two and wants the odd distance (d = 64, B16 H16 S2048: 243 against 257 us)
  constexpr int kLoopPadA = test_build::kLoopPadA >= 0 ? test_build::kLoopPadA : (FULLP && D == 64) ? 1 : 0;
  // (test build with time stamps: every wavefront records the shader clock at each barrier arrival and departure, in the
  // lanes of one register; lanes 62 and 63 take the constant-rate 100 MHz counter when the wavefront starts and ends,
  // which with the first and the last stamp gives the shader clock the kernel actually ran at)
  unsigned trace_reg = 0;
  int trace_n = 0;
  auto stamp = [&]() {
    if constexpr (test_build::kTraceTicks) {
      unsigned long long t;
      asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t) :: "memory");
      if (trace_n < 62)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tv_writelane_b32 %0, %1, m0" : "+v"(trace_reg) : "s"((unsigned)t), "s"(__builtin_amdgcn_readfirstlane(trace_n)));
      ++trace_n;
    }
  };
  auto stamp_real = [&](int slot) {
    if constexpr (test_build::kTraceTicks) {
      unsigned long long t;
      asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t) :: "memory");
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tv_writelane_b32 %0, %1, m0" : "+v"(trace_reg) : "s"((unsigned)t), "s"(slot));
    }
  };
  stamp();
  stamp_real(62);
  auto barrier = [&]() { stamp(); asm volatile("s_barrier" ::: "memory"); stamp(); };

  // One workgroup barrier per key block, or (a test build) two: see the schedule below.
  constexpr bool kOneBarrier = !test_build::kTwoBarriers;
  constexpr int kVAhead = (FULLP && kOneBarrier) ? 3 : 2;

  const int row0 = qb * kBlockQ + wave * 32;  // first query row of this wavefront
  const bool active = row0 < Sq;              // the last workgroup of a head may be partly empty

  // ---- state of a wavefront ----------------------------------------------------------------------------------------
  // (declared here, ahead of the code that uses it; given its start values by init_state(), which each half of the
  // workgroup calls once its first loads are on their way)
  float o_f[kDSteps][16];  // running O, not normalised
  float m_ref;             // reference exponent of the running O and l (base-2 units)
  float t_run;             // FASTACC: sum of the merge weights, i.e. how much of kBase the running O carries
  float l_run;             // running row sum, in units of 1/128 (it sums 128*p)
  bool merged_any = false; // some key block has been merged into O, l and t
  const float c2 = BIAS ? args.c2 * kBaseScale : args.c2;  // exponent per unit of sf() below
  constexpr int kScoreBaseBits = score_base_bits<D>();  // start value of the GEMM 1 accumulators on the BIAS variant
  const float bias_c2 = BIAS ? __builtin_bit_cast(float, kScoreBaseBits) * c2 : 0.f;
  float magic;
  int flip_top;
  v16i base_c;             // start value of the GEMM 2 accumulators (and of GEMM 1 at head_dim 128), in sixteen registers
  v16i base_s;             // start value of the GEMM 1 accumulators
  v4i qreg[kDSteps];       // Q: B operand of GEMM 1, loaded once
  int kb_end = 0;          // one past the last key block that holds any unmasked key (trailing padding is never computed on)
  int kb_plain = 0;        // the first block with any masked key: blocks [0, kb_plain) have none
  int n = 0, last = -1;    // kb_end and kb_end - 1 under the names the schedule uses
  unsigned tail_word[kKeyTiles];  // RAGGED: mask bits of the shifted last block
  auto init_state = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kDSteps; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r) o_f[u][r] = 0.f;
    m_ref = args.floor2 - 2.f * kLazyLog2;
    t_run = 0.f;
    l_run = 0.f;
    magic = kMagic;
    asm volatile("" : "+v"(magic));  // a register operand: as a literal it would double the size of every instruction using it
    flip_top = (int)0x80808080;
    if (FULLP) asm volatile("" : "+s"(flip_top));  // a register operand, for the same reason
    base_c = v16i{kBaseBits, kBaseBits, kBaseBits, kBaseBits, kBaseBits, kBaseBits, kBaseBits, kBaseBits,
                  kBaseBits, kBaseBits, kBaseBits, kBaseBits, kBaseBits, kBaseBits, kBaseBits, kBaseBits};
    asm volatile("" : "+v"(base_c));  // held in registers: as a known constant it is rebuilt by eight moves per key block
    if (kScoreBaseBits == kBaseBits) {
      base_s = base_c;
    } else {
      base_s = v16i{kScoreBaseBits, kScoreBaseBits, kScoreBaseBits, kScoreBaseBits, kScoreBaseBits, kScoreBaseBits,
                    kScoreBaseBits, kScoreBaseBits, kScoreBaseBits, kScoreBaseBits, kScoreBaseBits, kScoreBaseBits,
                    kScoreBaseBits, kScoreBaseBits, kScoreBaseBits, kScoreBaseBits};
      if (BIAS) asm volatile("" : "+v"(base_s));
    }
  };

  // ---- the prologue ------------------------------------------------------------------------------------------------
  // Its loads are all issued before any is waited for and all by inline assembly, so that every wait is an explicit
  // s_waitcnt vmcnt(n) that counts the loads still allowed in flight (memory reads return in issue order):
  //   wavefronts 0..3:  K0 (all of it) | mask bytes of the first 4096 keys (1 load) | Q (kDSteps loads)
  //   wavefronts 4..7:  Q (kDSteps loads) | behind the first barrier: V0 (all of it)
  // (the next tiles follow right after the first barrier: the CU's vector memory path moves 64 bytes per cycle, and
  // everything queued here delays the first GEMM.)  The first barrier publishes K0, which wavefronts 0..3 fetch alone:
  // it waits for nothing that wavefronts 4..7, which start several hundred cycles later, have asked for.  Each half of
  // the workgroup runs its own prologue and its own schedule behind ONE branch on the wavefront index, so that a load
  // and the wait that retires it always lie on the same path.
  auto load_q_rows = [&]() __attribute__((always_inline)) {
    // rows past the end of the sequence load the last row (unused) so that every wavefront has the same loads in flight
    const int8_t* qp = args.q + q_head_off;
    int qrow = row0 + i32 < Sq ? row0 + i32 : Sq - 1;
    if (!fmha_in_bounds(qrow >= 0 && qrow < Sq)) qrow = 0;
    const int qoff = qrow * D + 16 * g;
#pragma unroll
    for (int kk = 0; kk < kDSteps; ++kk)
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(qreg[kk]) : "v"(qoff + 32 * kk), "s"(qp) : "memory");
  };
  // The Q registers are redefined after the wait that retires their loads, so that no use of them can be scheduled
  // above it.
  auto pin_q_rows = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int kk = 0; kk < kDSteps; ++kk) asm volatile("" : "+v"(qreg[kk]));
  };
  // Wavefronts 0..3 also classify the key blocks of this batch entry, sixteen mask bytes per lane and BK/16 lanes per
  // block: their loads are the first to be served.  Per key block: lds_class (bit0 = some key masked, bit1 = all keys
  // masked) and the mask bits themselves (lds_mask); per classifying wavefront: the last block it saw with an unmasked
  // key and the first with a masked one (lds_scan).  All of it is published by the first barrier, together with K0.
  constexpr int kClassWaves = 4;
  constexpr int kKeysPerLane = 16;
  constexpr int kKeysPerPass = kKeysPerLane * 64 * kClassWaves;
  auto prologue_waves_0_to_3 = [&]() __attribute__((always_inline)) {
    issue_tile0_by_half(kg, 0, ld_goff_k);
    v4i mask_bytes = {0, 0, 0, 0};
    {
      const bool inside = kKeysPerLane * tid + kKeysPerLane <= S;
      int j = inside ? kKeysPerLane * tid : 0;
      if (!fmha_in_bounds(!inside || (j >= 0 && j + kKeysPerLane <= S))) j = 0;
      if (!RAGGED || S >= kKeysPerLane)  // (a shorter mask row has no 16 bytes that lie inside it)
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(mask_bytes) : "v"(j), "s"(mg) : "memory");
    }
    // RAGGED: the last sixteen mask bytes of the row, for the one lane whose sixteen keys straddle its end
    v4i tail_bytes = {0, 0, 0, 0};
    if (RAGGED && S >= kKeysPerLane) {
      int j = S - kKeysPerLane;
      if (!fmha_in_bounds(j >= 0 && j + kKeysPerLane <= S)) j = 0;
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(tail_bytes) : "v"(j), "s"(mg) : "memory");
    }
    load_q_rows();
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(mask_bytes) : "n"(kDSteps) : "memory");
    asm volatile("" : "+v"(tail_bytes));
    constexpr int kLanesPerBlock = BK / kKeysPerLane;
    constexpr int kBlocksPerWave = 64 / kLanesPerBlock;
    constexpr unsigned long long kGroupBits = kLanesPerBlock == 8 ? 0x0101010101010101ull : 0x1111111111111111ull;
    int live_hi = -1, pad_lo = 0x7fffffff;
    // one bit per byte of a dword: set where the byte is not zero
    auto nonzero_bytes = [](unsigned w) -> unsigned {
      const unsigned t = (((w & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w) & 0x80808080u;  // bit 7 of every nonzero byte
      return (((t >> 7) * 0x00204081u) >> 21) & 15u;                           // ... gathered into bits 0..3
    };
    for (int base = 0; base < S_pad; base += kKeysPerPass) {
      const int j = base + kKeysPerLane * tid;
      unsigned bits = 0xffffu;  // keys past the end of the sequence count as masked
      if (j + kKeysPerLane <= S) {
        v4i w = mask_bytes;
        if (base != 0) {
          const int jj = fmha_in_bounds(j >= 0 && j + kKeysPerLane <= S) ? j : 0;
          asm volatile("global_load_dwordx4 %0, %1, %2\n\ts_waitcnt vmcnt(0)" : "=v"(w) : "v"(jj), "s"(mg) : "memory");
        }
        bits = nonzero_bytes((unsigned)w[0]) | (nonzero_bytes((unsigned)w[1]) << 4) | (nonzero_bytes((unsigned)w[2]) << 8) |
               (nonzero_bytes((unsigned)w[3]) << 12);
      } else if (RAGGED && j < S) {  // the one lane that straddles the end
        if (S >= kKeysPerLane) {
          // its S - j keys are the last S - j of the row's last sixteen
          const unsigned last16 = nonzero_bytes((unsigned)tail_bytes[0]) | (nonzero_bytes((unsigned)tail_bytes[1]) << 4) |
                                  (nonzero_bytes((unsigned)tail_bytes[2]) << 8) | (nonzero_bytes((unsigned)tail_bytes[3]) << 12);
          bits = ((last16 >> (kKeysPerLane - (S - j))) | (0xffffu << (S - j))) & 0xffffu;
        } else {
          for (int b = 0; b < S - j; ++b) bits = (mg[fmha_in_bounds(j + b < S) ? j + b : 0] != 0) ? bits : (bits & ~(1u << b));
        }
      }
      // two lanes hold the 32 mask bits of one word
      const unsigned word = bits | ((unsigned)__shfl_xor((int)bits, 1) << 16);
      if ((lane & 1) == 0 && j < S_pad) lds_mask[j >> 5] = word;
      const unsigned long long some = __ballot(bits != 0), all = __ballot(bits == 0xffffu);
      if (lane % kLanesPerBlock == 0 && j < S_pad) {
        constexpr unsigned long long kBlockBits = (1ull << kLanesPerBlock) - 1;
        const unsigned long long blk_some = (some >> lane) & kBlockBits, blk_all = (all >> lane) & kBlockBits;
        lds_class[j / BK] = (unsigned char)((blk_some != 0 ? 1 : 0) | (blk_all == kBlockBits ? 2 : 0));
      }
      // the same two facts per block of this wavefront, folded onto the lowest lane of each block (wave-uniform)
      unsigned long long any = some, every = all;
#pragma unroll
      for (int sh = 1; sh < kLanesPerBlock; sh *= 2) {
        any |= any >> sh;
        every &= every >> sh;
      }
      const int blk0 = (base + kKeysPerLane * 64 * wave) / BK;  // first block of this wavefront in this pass
      const int n_here = min(max(n_blocks - blk0, 0), kBlocksPerWave);
      const unsigned long long valid = (n_here == kBlocksPerWave ? ~0ull : ((1ull << (n_here * kLanesPerBlock)) - 1ull)) & kGroupBits;
      const unsigned long long live = ~every & valid, padded = any & valid;
      if (live != 0) live_hi = blk0 + (63 - __builtin_clzll(live)) / kLanesPerBlock;
      if (padded != 0) pad_lo = min(pad_lo, blk0 + __builtin_ctzll(padded) / kLanesPerBlock);
    }
    if (lane == 0) {
      lds_scan[2 * wave] = live_hi;
      lds_scan[2 * wave + 1] = pad_lo;
    }
    init_state();
    // K0 and the Q rows have landed; the LDS writes above are not waited for by the hand-written barrier
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    pin_q_rows();
  };
  // Wavefronts 4..7 ask for their Q rows only and wait for nothing in front of the first barrier; right behind it they
  // wait for the Q rows (their first GEMM 1 comes one phase later anyway) and then ask for V0, which is first needed
  // behind the second barrier.  Every wait of the prologue is a vmcnt(0): it holds on whatever path leads to it.
  // (FULLP with one barrier per key block: V0 in front of the first barrier - they sum its columns right behind it.)
  constexpr bool kV0BeforeFirstBarrier = FULLP && kOneBarrier;
  auto prologue_waves_4_to_7 = [&]() __attribute__((always_inline)) {
    load_q_rows();
    if (kV0BeforeFirstBarrier) issue_tile0_by_half(vg, 1, ld_goff_v);
    init_state();
    if (kV0BeforeFirstBarrier) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      pin_q_rows();
    }
  };
  auto q_rows_landed_then_v0 = [&]() __attribute__((always_inline)) {  // wavefronts 4..7, behind the first barrier
    if (!kV0BeforeFirstBarrier) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      pin_q_rows();
      issue_tile0_by_half(vg, 1, ld_goff_v);
    }
  };
  // Barrier 0 publishes K0, the block classes, the mask bits and the scan records; every wavefront then reads what the
  // classification found.
  auto first_barrier = [&]() __attribute__((always_inline)) {
    prologue_done = true;
    barrier();
    {
      const v4i s0 = *reinterpret_cast<const v4i*>(&lds_scan[0]), s1 = *reinterpret_cast<const v4i*>(&lds_scan[4]);
      kb_end = __builtin_amdgcn_readfirstlane(max(max(s0[0], s0[2]), max(s1[0], s1[2]))) + 1;
      kb_plain = __builtin_amdgcn_readfirstlane(min(min(min(s0[1], s0[3]), min(s1[1], s1[3])), n_blocks));
    }
    n = kb_end;
    last = n - 1;
    // mask bits of the shifted last block: bit r of word t <-> key S - BK + 32 t + r; the repeated keys count as masked
#pragma unroll
    for (int t = 0; t < kKeyTiles; ++t) tail_word[t] = 0;
    if (RAGGED && tail_kb >= 0) {
      const int repeated = BK - tail_rows;
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        const int start = S - BK + 32 * t, w = start >> 5, sh = start & 31;
        const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_mask[w]);
        const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_mask[w + (sh ? 1 : 0)]);
        unsigned word = sh ? (lo >> sh) | (hi << (32 - sh)) : lo;
        const int forced = repeated - 32 * t;  // leading bits of this word that belong to repeated keys
        if (forced >= 32) word = 0xffffffffu;
        else if (forced > 0) word |= (1u << forced) - 1u;
        tail_word[t] = word;
      }
    }
  };

  // ---- the four phases of one key block ----------------------------------------------------------------------------
  // acc:  S^T, for query column i32 keys 32t + 8a + 4g + bb at acc[t][4a+bb]        (GEMM 1 -> softmax)
  // pk:   P^T, int8, B operand of GEMM 2                                              (softmax -> GEMM 2)
  // oacc: O~^T, output dims 32u + 8a + 4g + bb at oacc[u][4a+bb], as kBaseBits + O~   (GEMM 2 -> merge)
  float m_blk = 0.f;    // block-local row maximum, base-2 units
  float l_blk = 0.f;    // sum of (128/32767) p over this lane's keys

  // Row maximum of one finished 32-key tile, folded into two independent chains (integer compare: monotone in the
  // score, also for the biased bit patterns).  Four pieces of two instructions, one behind each MFMA of the next tile.
  auto tile_max_piece = [&](const v16i& a, int (&mx)[2], bool first, int j) __attribute__((always_inline)) {
    if (first && j == 0) {
      mx[0] = max(max(a[0], a[1]), a[2]);
      mx[1] = max(max(a[8], a[9]), a[10]);
    } else if (first) {
      mx[0] = (j < 3) ? max(max(mx[0], a[1 + 2 * j]), a[2 + 2 * j]) : max(mx[0], a[7]);
      mx[1] = (j < 3) ? max(max(mx[1], a[9 + 2 * j]), a[10 + 2 * j]) : max(mx[1], a[15]);
    } else {
      mx[0] = max(max(mx[0], a[2 * j]), a[2 * j + 1]);
      mx[1] = max(max(mx[1], a[8 + 2 * j]), a[9 + 2 * j]);
    }
  };

  // GEMM 1: S^T[key][query] = K . Q^T, int32 (inc/fmha_i8.cuh:120-172), one 32-key tile after the other; the row
  // maximum of tile t-1 is taken while the MFMAs of tile t run.  mx covers tiles 0 .. kKeyTiles-2 on return.
  //
  // masked = true: some keys of this block are masked out (nonzero mask byte, inc/fmha_i8.cuh:189-192,216-221).  The
  // ACCUMULATORS of a masked key start at a value that loses every maximum and whose exponential is exactly 0 whatever
  // the MFMAs add to it - read as a float on the BIAS variant, 0xFF000000 + S is below -2^126 for every |S| < 2^21;
  // where the scores are converted, -2^30 + S times that variant's c2 >= 2.7e-4 is an exponent below -2.9e5 - so that
  // the row maximum taken behind the MFMAs and the whole softmax need no further look at the mask.  The start values
  // are one v_cndmask per score on wave-uniform lane masks - lanes 0..31 hold key 8a+bb of a tile, lanes 32..63 key
  // 8a+4+bb, so the scalar unit builds them from the block's mask bits - written into the accumulator registers
  // themselves, tile by tile, in front of the tile's MFMAs.
  auto phase_gemm1 = [&](int kb, v16i (&acc)[kKeyTiles], int (&mx)[2], bool masked = false) __attribute__((always_inline)) {
    if constexpr (test_build::kNoMfma) {
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) test_build::undefined(acc[t]);
      test_build::undefined(mx[0]);
      test_build::undefined(mx[1]);
      return;
    }
    const int8_t* lds_k = &lds[kb & (kStages - 1)][0][0];
    const v16i zero_c = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    v4i ka[2][kDSteps];  // operand reads run one key tile ahead of the MFMAs that consume them
    auto read_k = [&](int off) {
      v4i operand;
      if constexpr (test_build::kNoLdsReads) test_build::undefined(operand);
      else operand = *reinterpret_cast<const v4i*>(lds_k + off);
      return operand;
    };
    unsigned mw[kKeyTiles];  // masked: the block's mask bits, bit j of word t <-> key 32 t + j of the block
    int gone = BIAS ? (int)0xFF000000 : -(1 << 30);
    if (masked) {
      asm volatile("" : "+v"(gone));  // a register operand
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t)
        mw[t] = (RAGGED && kb == tail_kb) ? tail_word[t]
                                          : (unsigned)__builtin_amdgcn_readfirstlane((int)lds_mask[kb * kKeyTiles + t]);
    }
    auto start_piece = [&](int t, int first, int count) __attribute__((always_inline)) {  // start values of registers first .. first+count-1 of tile t
#pragma unroll
      for (int r = first; r < first + count; ++r) {
        const int key = 8 * (r / 4) + (r % 4);
        const unsigned lo = (unsigned)(((int)(mw[t] << (31 - key))) >> 31), hi = (unsigned)(((int)(mw[t] << (27 - key))) >> 31);
        const unsigned long long lanes = ((unsigned long long)hi << 32) | lo;
        int e;
        if (BIAS) asm volatile("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(e) : "v"(base_s[0]), "v"(gone), "s"(lanes));
        else asm volatile("v_cndmask_b32_e64 %0, 0, %1, %2" : "=v"(e) : "v"(gone), "s"(lanes));
        acc[t][r] = e;
      }
    };
    if (masked) {
      // One operand buffer and no read-ahead: the start values of a tile are written while its operand reads are in
      // flight, and the registers that the read-ahead would take are what the accumulators of the next tile, live one
      // chain early here, need (with both, the d = 128 kernel spills).
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
#pragma unroll
        for (int kk = 0; kk < kDSteps; ++kk) ka[0][kk] = read_k(k_read_off[kk] + 32 * t * D);
        align8(true);
        start_piece(t, 0, 16);
        asm volatile("s_nop 1" ::: "memory");  // (the compiler does not know that the statements above wrote registers an MFMA reads)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < kDSteps; ++kk) {
          align8(true);
          acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[0][kk], qreg[kk], acc[t], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (t >= 1) {
#pragma unroll
            for (int j = kk * 4 / kDSteps; j < (kk + 1) * 4 / kDSteps; ++j) tile_max_piece(acc[t - 1], mx, t == 1, j);
            asm volatile("" : "+v"(mx[0]), "+v"(mx[1]));
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
      return;
    }
#pragma unroll
    for (int kk = 0; kk < kDSteps; ++kk) ka[0][kk] = read_k(k_read_off[kk]);
#pragma unroll
    for (int t = 0; t < kKeyTiles; ++t) {
      if (t + 1 < kKeyTiles) {
#pragma unroll
        for (int kk = 0; kk < kDSteps; ++kk)
          ka[(t + 1) & 1][kk] = read_k(k_read_off[kk] + 32 * (t + 1) * D);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < kDSteps; ++kk) {
        align8();
        acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[t & 1][kk], qreg[kk],
                                                       kk == 0 ? (BIAS ? base_s : zero_c) : acc[t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (t >= 1) {
#pragma unroll
          for (int j = kk * 4 / kDSteps; j < (kk + 1) * 4 / kDSteps; ++j) tile_max_piece(acc[t - 1], mx, t == 1, j);
          asm volatile("" : "+v"(mx[0]), "+v"(mx[1]));  // keeps these few instructions here, in the shadow of the MFMA
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  // (sf(t,r) below: the score as a float; with BIAS that is the start value + S * 2^-26, and the exponent offset removes the start value.)
  // block softmax (inc/fmha_i8.cuh:174-253)
  // split = false: the whole block softmax, P packed, software-pipelined (the general loop).  split = true (the
  // steady-state loop): everything but the P packing, in three dense runs - 64 scale fmas, 64 exponentials, 64 + 4 adds -
  // and the exponentials are left in acc (as float bits) for phase_pack, which runs at the head of the MFMA phase.
  auto phase_softmax = [&](int kb, int cls, v16i (&acc)[kKeyTiles], v4i (&pk)[kKeyTiles], int (&mx)[2], bool split = false, bool aligned = false) __attribute__((always_inline)) {
    if constexpr (test_build::kNoSoftmax) {
      if (!split) {
#pragma unroll
        for (int t = 0; t < kKeyTiles; ++t) test_build::undefined(pk[t]);
      }
      test_build::undefined(m_blk);
      test_build::undefined(l_blk);
      return;
    }
    auto sf = [&](int t, int r) -> float { return BIAS ? __int_as_float(acc[t][r]) : (float)acc[t][r]; };
    l_blk = 0.f;
    // (cls != 0: some keys of this block are masked out.  GEMM 1 has seen to it that their scores lose every maximum
    // and that their exponentials are exactly 0; what is left to do here is the reference's sentinel, below.)
    {
#pragma unroll
      for (int j = 0; j < 4; ++j) tile_max_piece(acc[kKeyTiles - 1], mx, false, j);
      int ti = half_max(max(mx[0], mx[1]));
      // a masked key enters the maximum as the integer -1000000 (inc/fmha_i8.cuh:191-193)
      if (cls != 0) ti = max(ti, (BIAS ? kScoreBaseBits : 0) - 1000000);
      const float top = BIAS ? __int_as_float(ti) : (float)ti;
      // off = top*c2 rounded; p' = exp2(s*c2 - off) = p * 2^(resid) with one row-wide resid below 1 ulp of off, and the
      // block maximum that is consistent with p' is off itself (minus the constant kBase*c2 when BIAS).
      float off = top * c2;
      // Where the scores are converted, c2 is large and |off| can reach 10^5 and more: the rounding of this product and
      // of offq below then amounts to a percent of p, and a p above 1 by 0.4 % quantises to -129, whose low byte is
      // +127.  Two units in the last place upwards make off an upper bound of the exact product: every p is at most 1,
      // the row is scaled by one common factor just below 1 (l with it: the output does not notice).
      if (!BIAS) off = __builtin_fmaf(fabsf(off), 2.384185791015625e-07f, off);
      if (!BIAS) off = fmaxf(off, args.floor2);
      m_blk = off - bias_c2;
      // exp2(x - offq) = 128 p / 32767: the snorm conversion returns rne(128 p) (FULLP: 255 in place of 128)
      const float offq = off - (FULLP ? kLog2PscaleFull : kLog2Pscale);
      // Software pipeline over quads of four scores (quad qd = 4 t + a): step s issues the four exponentials of quad s
      // with the four scaling fmas of quad s+1 and the sums and packing of quad s-1 between them.  A wavefront issues in
      // order, a transcendental occupies its unit for about two issue slots, and an instruction that follows one without
      // needing the unit goes out in its shadow; the fences make the scheduler keep this order.
      constexpr int kQuads = 4 * kKeyTiles;
      if (split) {
        // The same arithmetic in the same order of additions as the pipeline below, instruction class by instruction
        // class: measured against the pipelined form with the packing left to the compiler's placement, -6 % at d = 64
        // (where it also makes one barrier per key block the faster choice) and level at d = 128.
        float xs[kQuads][4];
        align8(aligned);
#pragma unroll
        for (int qd = 0; qd < kQuads; ++qd)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            xs[qd][j] = test_build::kNoScaleRun ? __int_as_float(acc[qd / 4][4 * (qd % 4) + j])
                                                : __builtin_fmaf(sf(qd / 4, 4 * (qd % 4) + j), c2, -offq);
#pragma unroll
        for (int qd = 0; qd < kQuads; ++qd) asm volatile("" : "+v"(xs[qd][0]), "+v"(xs[qd][1]), "+v"(xs[qd][2]), "+v"(xs[qd][3]));
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!test_build::kNoExpRun) {
#pragma unroll
          for (int qd = 0; qd < kQuads; ++qd)
#pragma unroll
            for (int j = 0; j < 4; ++j) xs[qd][j] = __builtin_amdgcn_exp2f(xs[qd][j]);
        }
#pragma unroll
        for (int qd = 0; qd < kQuads; ++qd) asm volatile("" : "+v"(xs[qd][0]), "+v"(xs[qd][1]), "+v"(xs[qd][2]), "+v"(xs[qd][3]));
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (test_build::kMfmaRowSum) {
          // (test build: the row sum on the matrix pipe.  The exponentials are rounded to half precision two at a time
          // and eight of them per lane go into one v_mfma_f32_16x16x32_f16 as the B operand - lane l brings eight keys
          // of query l%32, so column n of B holds query n in the k-slots of lanes n and n+32 and query n+16 in those of
          // lanes n+16 and n+48 - against an A operand whose rows 0..3 and 8..11 are 1 on the first kind of k-slot and 0
          // on the second, rows 4..7 and 12..15 the other way round: every lane then receives, four times, the sum over
          // both lanes of its own query.  32 conversions and 8 MFMAs in place of 67 additions and the lane exchange.)
          typedef float f2 __attribute__((ext_vector_type(2)));
          typedef float f4 __attribute__((ext_vector_type(4)));
          typedef _Float16 h2 __attribute__((ext_vector_type(2)));
          typedef _Float16 h8 __attribute__((ext_vector_type(8)));
          const _Float16 one = ((((lane & 15) >> 2) ^ (lane >> 4)) & 1) ? (_Float16)0.f : (_Float16)1.f;
          const h8 ones = {one, one, one, one, one, one, one, one};
          f4 lsum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int qd = 0; qd < kQuads; qd += 2) {
            const h2 p0 = __builtin_convertvector(f2{xs[qd][0], xs[qd][1]}, h2), p1 = __builtin_convertvector(f2{xs[qd][2], xs[qd][3]}, h2);
            const h2 p2 = __builtin_convertvector(f2{xs[qd + 1][0], xs[qd + 1][1]}, h2), p3 = __builtin_convertvector(f2{xs[qd + 1][2], xs[qd + 1][3]}, h2);
            const h8 b = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
            lsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, b, lsum, 0, 0, 0);
          }
#pragma unroll
          for (int qd = 0; qd < kQuads; ++qd)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[qd / 4][4 * (qd % 4) + j] = __float_as_int(xs[qd][j]);
          l_blk = lsum[0];
          return;
        }
#pragma unroll
        for (int qd = 0; qd < kQuads; ++qd) {
          if constexpr (test_build::kNoSumRun) {
            if (qd == 0) l_blk += xs[0][0];
          } else {
            float s01 = xs[qd][0] + xs[qd][1];
            const float s23 = xs[qd][2] + xs[qd][3];
            s01 += s23;
            l_blk += s01;
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[qd / 4][4 * (qd % 4) + j] = __float_as_int(xs[qd][j]);
        }
        l_blk = half_sum(l_blk);
        return;
      }
      float x[3][4];  // x[qd % 3]: scaled exponents, then exponentials, of quad qd
      auto q_fma = [&](int qd, int j) {
        x[qd % 3][j] = __builtin_fmaf(sf(qd / 4, 4 * (qd % 4) + j), c2, -offq);
      };
      auto q_exp = [&](int qd, int j) { x[qd % 3][j] = __builtin_amdgcn_exp2f(x[qd % 3][j]); };
      float s01 = 0.f, s23 = 0.f;
      v2s lo, hi;
      auto q_out = [&](int qd, int j) {  // seven steps of sums and packing of quad qd
        const float(&e)[4] = x[qd % 3];
        if (j == 0) s01 = e[0] + e[1];
        if (j == 1) s23 = e[2] + e[3];
        if (j == 2) lo = FULLP ? __builtin_amdgcn_cvt_pknorm_i16(e[0], e[1]) : __builtin_amdgcn_cvt_pknorm_i16(-e[0], -e[1]);
        if (j == 3) hi = FULLP ? __builtin_amdgcn_cvt_pknorm_i16(e[2], e[3]) : __builtin_amdgcn_cvt_pknorm_i16(-e[2], -e[3]);
        if (j == 4) s01 += s23;
        if (j == 5) {
          const int four = __builtin_amdgcn_perm(__builtin_bit_cast(int, hi), __builtin_bit_cast(int, lo), 0x06040200);
          pk[qd / 4][qd % 4] = FULLP ? four ^ flip_top : four;  // FULLP: the bytes 0..255 become P - 128
        }
        if (j == 6) l_blk += s01;
      };
      if (kQuads > 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) q_fma(0, j);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int s = 0; s <= kQuads; ++s) {
        const bool ex = s < kQuads, fm = s + 1 < kQuads, out = s >= 1;
        auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
        if (ex) { q_exp(s, 0); fence(); }
        if (fm) { q_fma(s + 1, 0); q_fma(s + 1, 1); }
        if (out) q_out(s - 1, 0);
        fence();
        if (ex) { q_exp(s, 1); fence(); }
        if (fm) { q_fma(s + 1, 2); q_fma(s + 1, 3); }
        if (out) q_out(s - 1, 1);
        fence();
        if (ex) { q_exp(s, 2); fence(); }
        if (out) { q_out(s - 1, 2); q_out(s - 1, 3); q_out(s - 1, 4); }
        fence();
        if (ex) { q_exp(s, 3); fence(); }
        if (out) { q_out(s - 1, 5); q_out(s - 1, 6); }
        fence();
      }
      l_blk = half_sum(l_blk);
    }
  };
  // P packing of the exponentials that phase_softmax(split) left in acc: P^T as the B operand of GEMM 2.
  auto phase_pack = [&](v16i (&acc)[kKeyTiles], v4i (&pk)[kKeyTiles], bool aligned = false) __attribute__((always_inline)) {
    if constexpr (test_build::kNoSoftmax) {
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) test_build::undefined(pk[t]);
      return;
    }
    align8(aligned);
#pragma unroll
    for (int qd = 0; qd < 4 * kKeyTiles; ++qd) {
      float e[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) e[j] = __int_as_float(acc[qd / 4][4 * (qd % 4) + j]);
      const v2s lo = FULLP ? __builtin_amdgcn_cvt_pknorm_i16(e[0], e[1]) : __builtin_amdgcn_cvt_pknorm_i16(-e[0], -e[1]);
      const v2s hi = FULLP ? __builtin_amdgcn_cvt_pknorm_i16(e[2], e[3]) : __builtin_amdgcn_cvt_pknorm_i16(-e[2], -e[3]);
      const int four = __builtin_amdgcn_perm(__builtin_bit_cast(int, hi), __builtin_bit_cast(int, lo), 0x06040200);
      pk[qd / 4][qd % 4] = FULLP ? four ^ flip_top : four;  // FULLP: the bytes 0..255 become P - 128
    }
  };
  // The results of a split softmax are pinned where the source has them - before the barrier - and the packing behind
  // the raised priority: left alone, the compiler moves both (none of them touches memory).
  // The steady-state loop uses the split form: -6 % at d = 64 (where it also makes one barrier per key block the faster
  // choice), -2 % at d = 128 and S = 4096 against the pipelined form, whose packing the compiler places by itself.
  constexpr bool kSplitSoftmax = true;
  auto pin_scores = [&](v16i (&acc)[kKeyTiles]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < kKeyTiles; ++t) asm volatile("" : "+v"(acc[t]));
    asm volatile("" : "+v"(l_blk), "+v"(m_blk));
  };

  // GEMM 2 and the online merge in one phase.  O~^T[d][query] = V^T . P^T, int32 (inc/fmha_i8.cuh:255-296), one
  // 32-row output tile u after the other (accumulators start at kBaseBits), and tile u-1 is merged into the running O
  // (inc/fmha_i8.cuh:298-315) four elements behind each MFMA of tile u.  Normalisation is deferred to the epilogue:
  // O and l are kept relative to 2^m_ref, and m_ref only moves when some row's block maximum exceeds it by
  // 2^kLazyLog2.
  // Where the tile loads of a block are issued: one per output tile inside GEMM 2.  The loads and their address
  // arithmetic stand in the issue stream of whichever wavefront carries them; inside the MFMA phase they fall into the
  // waits of the MFMA chain (-7 % at d = 64 against issuing them after the softmax, -0.6 % at d = 128 against issuing them
  // in front of the MFMA phase).  The other placements are kept for the test build that stages the tiles through
  // registers, which needs the loads of a key block in one place.
  constexpr bool kLoadsInMfmaPhase = !test_build::kStagedLoads || D == 64;
  static_assert(!kLoadsInMfmaPhase || 2 * kRegionsPerWave <= kDSteps, "one tile load per output tile of GEMM 2");
  auto phase_gemm2_merge = [&](int kb, const v4i (&pk)[kKeyTiles], int k_next, int v_next, bool steady = false) __attribute__((always_inline)) {
    if constexpr (test_build::kNoMfma) {
      if (kLoadsInMfmaPhase) {
        issue_k(k_next);
        issue_v(v_next);
      }
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) test_build::consume(pk[t]);  // (the softmax that produced these stays)
      test_build::consume(m_blk);
      test_build::consume(l_blk);
      return;
    }
    if (__ballot(m_blk > m_ref + kLazyLog2) != 0) {
      const float m_new = fmaxf(m_ref, m_blk);
      const float keep = __builtin_amdgcn_exp2f(m_ref - m_new);
      m_ref = m_new;
      if (merged_any) {  // (the first block always comes here, and has nothing to rescale: O, l and t are still 0)
        l_run *= keep;
        if (FASTACC) t_run *= keep;
#pragma unroll
        for (int u = 0; u < kDSteps; ++u)
#pragma unroll
          for (int r = 0; r < 16; ++r) o_f[u][r] *= keep;
      }
    }
    merged_any = true;
    const float take = __builtin_amdgcn_exp2f(m_blk - m_ref);
    l_run = __builtin_fmaf(take, l_blk, l_run);
    if (FASTACC) t_run += take;
    float neg_take = FULLP ? take : -take;  // P carries the sign: P = -128 p (inc/fmha_i8.cuh:298); FULLP: P = 255 p
    asm volatile("" : "+v"(neg_take));  // a plain register operand: as a source modifier it would force the 64-bit encoding
    auto merge_piece = [&](const v16i& oa, int u, int j) __attribute__((always_inline)) {  // four of the sixteen elements of output tile u
#pragma unroll
      for (int r = 4 * j; r < 4 * j + 4; ++r)
        o_f[u][r] = __builtin_fmaf(neg_take, FASTACC ? __int_as_float(oa[r]) : __int_as_float(oa[r]) - (FULLP ? kBaseFull : kBase),
                                   o_f[u][r]);
    };

    const int8_t* lds_v = &lds[kb & (kStages - 1)][1][0];
    typedef v2i __attribute__((address_space(3))) * lds_v2i_ptr;
    v2i va[2][kKeyTiles][2];  // transposed V operands of one output tile (all key tiles), one output tile ahead
    // FULLP: the accumulators of tile u start at what wavefronts 4..7 left in LDS for this key block (four 128-bit
    // reads per tile, fetched one tile ahead like the operands: a third buffer, since tile u-1 is still being merged)
    constexpr int kOaccBufs = FULLP ? 3 : 2;
    v16i oacc[kOaccBufs];
    auto ob = [&](int u) { return FULLP ? u % 3 : u & 1; };
    auto read_start = [&](int u) __attribute__((always_inline)) {
      const int* cs = &lds_colsum[(kb & 1) * D + 32 * u + 4 * g];
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const v4i w = *reinterpret_cast<const v4i*>(cs + 8 * a);
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) oacc[ob(u)][4 * a + bb] = w[bb];
      }
    };
    auto read_tile = [&](int u) __attribute__((always_inline)) {
      if constexpr (test_build::kNoLdsReads) {
#pragma unroll
        for (int t = 0; t < kKeyTiles; ++t) {
          test_build::undefined(va[u & 1][t][0]);
          test_build::undefined(va[u & 1][t][1]);
        }
        return;
      }
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        va[u & 1][t][0] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(lds_v + v_read_off[u] + 32 * t * D));
        va[u & 1][t][1] =
            __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(lds_v + v_read_off[u] + 32 * t * D + 16 * D));
      }
    };
    if (FULLP) read_start(0);
    read_tile(0);
#pragma unroll
    for (int u = 0; u < kDSteps; ++u) {
      if (u + 1 < kDSteps) {
        read_tile(u + 1);
        if (FULLP) read_start(u + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        const v4i a = {va[u & 1][t][0][0], va[u & 1][t][0][1], va[u & 1][t][1][0], va[u & 1][t][1][1]};
        oacc[ob(u)] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, pk[t], (t == 0 && !FULLP) ? base_c : oacc[ob(u)], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (u >= 1) {
#pragma unroll
          for (int j = t * 4 / kKeyTiles; j < (t + 1) * 4 / kKeyTiles; ++j) merge_piece(oacc[ob(u - 1)], u - 1, j);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (kLoadsInMfmaPhase) {
        if (u < kRegionsPerWave) issue_region(kg, k_next, 0, ld_goff_k, u, steady);
        else if (u < 2 * kRegionsPerWave) issue_region(vg, v_next, 1, ld_goff_v, u - kRegionsPerWave, steady);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) merge_piece(oacc[ob(kDSteps - 1)], kDSteps - 1, j);
  };
  // FULLP, wavefronts 4..7 (wavefront 4 + u: output tile u): the start values of GEMM 2 of key block kb.  The operand
  // reads of GEMM 2 hand lane (i32, g) sixteen keys of column 32u + i32 per key tile; v_dot4 against four ones sums
  // them, the two halves of the wavefront add up to the whole tile.  Rows of a tile that stand for keys which do not
  // exist (a ragged end) are counted like any other: their P is 0, i.e. the byte -128, and the two cancel.
  auto phase_colsum = [&](int kb) __attribute__((always_inline)) {
    if (colsum_tile >= 0 && colsum_tile < kDSteps) {
      const int8_t* lds_v = &lds[kb & (kStages - 1)][1][0];
      typedef v2i __attribute__((address_space(3))) * lds_v2i_ptr;
      int sum = 0;
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const v2i w = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(lds_v + colsum_read_off + 32 * t * D + 16 * D * h));
          sum = __builtin_amdgcn_sdot4(w[0], 0x01010101, sum, false);
          sum = __builtin_amdgcn_sdot4(w[1], 0x01010101, sum, false);
        }
      const auto r = __builtin_amdgcn_permlane32_swap(sum, sum, false, false);
      lds_colsum[(kb & 1) * D + 32 * colsum_tile + i32] = kBaseBitsFull + 128 * ((int)r[0] + (int)r[1]);
    }
  };
  // An LDS write is not waited for by the hand-written barrier: wavefronts 4..7 do so at the end of the phase.
  auto colsum_written = [&]() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };

  // ---- the schedule ------------------------------------------------------------------------------------------------
  // Every key block i is two phases per wavefront: an MFMA phase M(i) = [P packing and GEMM 2 + merge of block i]
  // [GEMM 1 of block i+1] and a VALU phase Y(i) = softmax of block i.  The two wavefronts of a SIMD run them in
  // anti-phase, so that the MFMA phase of one overlaps the VALU phase of the other.  They share one issue port: a key
  // block lasts about as long as the issue time of both phases of both wavefronts together, and the barrier waits for
  // the wavefront whose own instruction stream - vector, scalar and memory instructions alike - is the longer one.
  // ONE workgroup barrier per key block (numbered as the even ones of the two-barrier schedule below): between
  // barriers 2i+2 and 2i+4 wavefronts 0..3 run M(i) Y(i+1) and wavefronts 4..7 run Y(i) M(i).
  // Tiles: K(j), V(j) live in stage j mod 4; barrier 2m publishes K(m) and V(m-1), the operands of M(m-1) behind it.  K(i+3) and V(i+2) are requested inside M(i), one load behind each output
  // tile of GEMM 2 (a wavefront that issues loads is held for hundreds of cycles - the CU's vector memory path takes
  // 64 bytes per cycle and all eight wavefronts queue up - and there the hold falls into the waits of the MFMA chain);
  // their stages held K(i-1) and V(i-2), last read in M(i-2), which ends before barrier 2i.  Issue order per
  // wavefront: K0 V0 | K1 K2 V1 | K3 V2 | K4 V3 | ...
  // FULLP at d = 128: wavefronts 4..7 sum the columns of V(i+1) inside M(i), before their GEMM 1 of that block, and
  // the sums are read in M(i+1) by everyone, behind barrier 2i+4.  V therefore runs one key block further ahead than K
  // needs (the four V stages hold V(i) .. V(i+3)): barrier 2m publishes K(m) and V(m) instead of K(m) and V(m-1), and
  // the first barrier V(0).  Issue order per wavefront: K0 V0 | K1 V1 K2 V2 | K3 V3 | K4 V4 | ...
  // TWO barriers per key block (FULLP at d = 64, and the test build FMHA_TWO_BARRIERS): a tick is the interval between
  // two barriers; wavefronts 0..3 run M in even ticks and Y in odd ones, wavefronts 4..7 one tick behind.  The odd
  // barriers publish no tile; with FULLP barrier 2m+1 publishes the column sums of V(m), taken in tick 2m+1, and V runs
  // no further ahead than without FULLP.  Where the tile loads are not issued inside the MFMA phase (the staged test
  // build), wavefronts 0..3 issue theirs right after the barrier, in front of their MFMA phase, like wavefronts 4..7.
  auto barrier_odd = [&]() { if (!kOneBarrier) barrier(); };
  auto cls_of = [&](int kb) { return __builtin_amdgcn_readfirstlane((int)lds_class[kb]); };
  auto works = [&](int kb) { return active && !(cls_of(kb) & 2); };  // nothing in a fully masked block is attended to
  // Every issue point issues the same number of tiles whatever the position in the sequence: a tile index past the
  // last block is replaced by the last block, which is then fetched again into the stage it already occupies (the
  // same bytes: harmless for the wavefronts reading it).  That keeps the wait counts below compile-time constants and
  // the key loop free of the compares and branches that a count depending on the position would need.
  auto issue_first = [&]() __attribute__((always_inline)) {          // after barrier 0
    if (n > 0) {
      if (FULLP && kOneBarrier) {  // in pairs, so that "all but the newest two tiles" means the same at every barrier
        issue_k(min(1, last));
        issue_v(min(1, last));
        issue_k(min(2, last));
        issue_v(min(2, last));
      } else {
        issue_k(min(1, last));
        issue_k(min(2, last));
        issue_v(min(1, last));
      }
    }
  };
  auto issue_for = [&](int i) __attribute__((always_inline)) {  // where GEMM 2 of block i is skipped
    issue_k(min(i + 3, last));
    issue_v(min(i + kVAhead, last));
  };
  // Before barrier 2m every wavefront waits for its share of K(m) and V(m-1).  The tiles issued since may stay in
  // flight: the pair of the previous issue point and, for wavefronts 0..3 when they issue after the softmax (they
  // have just done so), the pair of this one.
  auto wait_tiles = [&](bool issued_after_softmax) {
    wait_all_but(!kLoadsInMfmaPhase && !kOneBarrier && issued_after_softmax ? 4 : 2);
  };
  auto issue_after_softmax = [&](int i) { if (!kLoadsInMfmaPhase) issue_for(i); };
  // wavefronts 0..3: the same pair of tiles either after the softmax or, with one barrier per key block, after the
  // barrier that follows it
  auto issue_after_softmax_a = [&](int i) { if (!kOneBarrier) issue_after_softmax(i); };
  auto issue_after_barrier_a = [&](int i) { if (kOneBarrier) issue_after_softmax(i); };
  // (test build that stages the tiles of the steady-state loop through registers, the "before" of the direct-to-LDS
  // loads: staged_step(i) loads the pair of tiles of issue point i into registers and writes the pair of issue point
  // i-1 to LDS.  The definitions live with the other test builds; in the shipped library kStaged is false and the three
  // calls are empty.)
  FMHA_STAGED_LOAD_LAMBDAS
  // FULLP with two barriers per key block: V(m) is summed by wavefronts 4..7 in tick 2m+1, one tick before its GEMM 2,
  // so it is barrier 2m+1 that publishes it.  Wavefronts 0..3 arrive there from their MFMA phase (the pair issued last may stay in flight),
  // wavefronts 4..7 from their softmax (the pair they have just issued; none where the loads go out in the MFMA phase).
  auto wait_v_for_colsum_a = [&]() { if (FULLP && !kOneBarrier) wait_all_but(2); };
  auto wait_v_for_colsum_b = [&]() { if (FULLP && !kOneBarrier) wait_all_but(kLoadsInMfmaPhase ? 0 : 2); };
  auto issue_in_mfma_phase = [&](int i) { if (kLoadsInMfmaPhase) issue_for(i); };
  v16i acc[kKeyTiles];  // S^T of the block whose softmax comes next (GEMM 1 -> softmax, across a barrier)
  int mx[2];
  // Where GEMM 1 is skipped the old scores are dead; saying so (an empty definition) keeps 64 registers from being
  // carried through the following MFMA phase.
  auto forget_scores = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < kKeyTiles; ++t) asm volatile("" : "=v"(acc[t]));
    asm volatile("" : "=v"(mx[0]), "=v"(mx[1]));
  };
  auto gemm1_of = [&](int kb) __attribute__((always_inline)) {  // GEMM 1 of block 0, which may or may not have masked keys
    if (cls_of(kb) != 0) phase_gemm1(kb, acc, mx, true);
    else phase_gemm1(kb, acc, mx, false);
  };
  // The wavefront in its MFMA phase gets the issue slots it asks for: an MFMA, an operand read or a merge instruction
  // that waits behind the other wavefront's softmax stream leaves the MFMA pipe idle, the reverse costs nothing.
  auto raise_priority = [&]() { asm volatile("s_setprio 3" ::: "memory"); };
  // Outside the MFMA phase wavefronts 0..3 run at priority 0.  Wavefronts 4..7 keep priority 1 there in the d = 64 kernel
  // that reads its scores without a conversion: when both wavefronts of a SIMD are in the softmax the older one (0..3)
  // otherwise wins every issue slot, and the workgroup starts with 4..7 behind.  Measured: B8 H12 S512 9.87 -> 9.57 us,
  // B32 H12 S256 13.15 -> 12.38, B64 H12 S384 45.7 -> 43.7, S2048 level; the converting d = 64 kernel loses 2 to 6 % from
  // 1024 keys on and the d = 128 kernels move by less than 1 % either way, so they stay at 0.  (Levels 1, 2 and 3
  // measure the same; the instruction has one length, so no code moves.)
  constexpr int kSoftmaxPriority47 = (D == 64 && BIAS) ? 1 : 0;
  auto drop_priority = [&]() {
    if (kSoftmaxPriority47 != 0 && wave >= kClassWaves) asm volatile("s_setprio %0" :: "n"(kSoftmaxPriority47) : "memory");
    else asm volatile("s_setprio 0" ::: "memory");
  };
  if (wave < kClassWaves) {
    prologue_waves_0_to_3();
    first_barrier();
    if (n > 0 && works(0)) gemm1_of(0);
    else forget_scores();
    issue_first();
    int i = 0;
    // Steady state, as long as blocks i and i+1 exist and have no masked key: the same phases as the general loop
    // below with every decision taken (scalar compares and branches are not free: they stand in the issue stream of
    // the wavefront that the barrier is waiting for).  A second loop of the same shape serves blocks with masked keys:
    // what it adds is the reference's sentinel in the softmax and the GEMM 1 that starts masked keys at "gone" (for
    // every block from the first one with a masked key on, whether the block has one or not: a branch between the
    // two forms of GEMM 1 inside the loop makes the d = 128 kernel spill).  Blocks whose keys are all masked, and the
    // last block, are left to the general loop.
    auto steady_a = [&](int i, int cls, bool next_masked) __attribute__((always_inline)) {
      v4i pk[kKeyTiles];
      wait_v_for_colsum_a();
      barrier_odd();
      phase_softmax(i, cls, acc, pk, mx, kSplitSoftmax, next_masked);
      if (kSplitSoftmax) pin_scores(acc);
      issue_after_softmax_a(i);
      staged_writes_done();
      wait_tiles(true);
      barrier();
      if (kStaged) staged_step(i);
      else issue_after_barrier_a(i);
      raise_priority();
      if (kSplitSoftmax) {
        pin_scores(acc);
        phase_pack(acc, pk, next_masked);
      }
      phase_gemm2_merge(i, pk, min(i + 3, last), min(i + kVAhead, last), true);
      if (next_masked) phase_gemm1(i + 1, acc, mx, true);
      else phase_gemm1(i + 1, acc, mx, false);
      drop_priority();
    };
    if (active) {
      align_loop();
      asm volatile(".rept %0\n\ts_nop 0\n\t.endr" :: "n"(kLoopPadA) : "memory");
      for (; i + 1 < n && i + 1 < kb_plain; ++i) steady_a(i, 0, false);
      if (!kStaged) {
        int cls = i < n ? cls_of(i) : 2;
        while (i + 1 < n && !(cls & 2)) {
          const int cls_next = cls_of(i + 1);
          if (cls_next & 2) break;
          steady_a(i, cls, true);
          cls = cls_next;
          ++i;
        }
      }
      if (kStaged) {
        staged_write();
        staged_writes_done();
      }
    }
    for (; i < n; ++i) {
      const int cls = cls_of(i);
      const bool work = active && !(cls & 2);
      v4i pk[kKeyTiles];
      wait_v_for_colsum_a();
      barrier_odd();                           // barrier 2i+1
      if (work) phase_softmax(i, cls, acc, pk, mx);
      issue_after_softmax_a(i);
      wait_tiles(true);
      barrier();                               // barrier 2i+2
      issue_after_barrier_a(i);
      raise_priority();
      if (work) phase_gemm2_merge(i, pk, min(i + 3, last), min(i + kVAhead, last));
      else issue_in_mfma_phase(i);
      if (i + 1 < n && works(i + 1)) phase_gemm1(i + 1, acc, mx, true);
      else forget_scores();
      drop_priority();
    }
    barrier_odd();                             // barrier 2n+1: wavefronts 4..7 run their last MFMA phase after it
  } else {
    prologue_waves_4_to_7();
    first_barrier();
    q_rows_landed_then_v0();
    issue_first();
    if (FULLP && !kOneBarrier) wait_all_but(3);  // V(0) has landed: K1 K2 V1 may be in flight
    barrier_odd();                             // barrier 1
    if (FULLP && n > 0) phase_colsum(0);
    if (n > 0 && works(0)) gemm1_of(0);
    else forget_scores();
    if (FULLP) colsum_written();
    int i = 0;
    auto steady_b = [&](int i, int cls, bool next_masked) __attribute__((always_inline)) {  // see steady_a above
      v4i pk[kKeyTiles];
      wait_tiles(false);
      barrier();
      phase_softmax(i, cls, acc, pk, mx, kSplitSoftmax, next_masked);
      if (kSplitSoftmax) pin_scores(acc);
      if (kStaged) staged_step(i);
      else issue_after_softmax(i);
      wait_v_for_colsum_b();
      barrier_odd();
      raise_priority();
      if (kSplitSoftmax) {
        pin_scores(acc);
        phase_pack(acc, pk, next_masked);
      }
      phase_gemm2_merge(i, pk, min(i + 3, last), min(i + kVAhead, last), true);
      if (FULLP) phase_colsum(i + 1);
      if (next_masked) phase_gemm1(i + 1, acc, mx, true);
      else phase_gemm1(i + 1, acc, mx, false);
      if (FULLP) colsum_written();
      drop_priority();
      staged_writes_done();
    };
    if (active) {
      align_loop();
      for (; i + 1 < n && i + 1 < kb_plain; ++i) steady_b(i, 0, false);
      if (!kStaged) {
        int cls = i < n ? cls_of(i) : 2;
        while (i + 1 < n && !(cls & 2)) {
          const int cls_next = cls_of(i + 1);
          if (cls_next & 2) break;
          steady_b(i, cls, true);
          cls = cls_next;
          ++i;
        }
      }
      if (kStaged) {
        staged_write();
        staged_writes_done();
      }
    }
    for (; i < n; ++i) {
      const int cls = cls_of(i);
      const bool work = active && !(cls & 2);
      v4i pk[kKeyTiles];
      wait_tiles(false);
      barrier();                               // barrier 2i+2
      if (work) phase_softmax(i, cls, acc, pk, mx);
      issue_after_softmax(i);
      wait_v_for_colsum_b();
      barrier_odd();                           // barrier 2i+3
      raise_priority();
      if (work) phase_gemm2_merge(i, pk, min(i + 3, last), min(i + kVAhead, last));
      else issue_in_mfma_phase(i);
      if (FULLP && i + 1 < n) phase_colsum(i + 1);
      if (i + 1 < n && works(i + 1)) phase_gemm1(i + 1, acc, mx, true);
      else forget_scores();
      if (FULLP) colsum_written();
      drop_priority();
    }
  }
  wait_all();  // nothing may still be writing LDS when the wavefront ends (only possible when every key is masked)
  stamp();
  stamp_real(63);
  test_build::write_trace(blockIdx.x, wave, lane, trace_reg);
  if (!active) return;

  // ---- epilogue: normalise, requantise, store (inc/fmha_i8.cuh:318-332) --------------------------------------------
  // l_run sums 128 p / 32767 and O sums 128 p v, so mean(v) = O / (32767 l_run); a row with no unmasked key yields 0
  const float fin = (l_run > 0.f) ? args.out_scale * (128.f / kSnorm) * kBaseScale / l_run : 0.f;
  const float corr = FASTACC ? (FULLP ? -kBaseFull * t_run : kBase * t_run) : 0.f;
  float magic_lo = kMagic - 127.f, magic_hi = kMagic + 127.f;
  asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));  // register operands, like magic
  int w[kDSteps][4];  // w[u][a]: the four int8 of output dims 32u + 8a + 4g .. +3 of query row i32
#pragma unroll
  for (int u = 0; u < kDSteps; ++u)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      float y[4];
#pragma unroll
      // magic + y holds rne(y) in the low mantissa bits (round-half-even): one fma rounds the scaled output once, and
      // the clamp to [-127, 127] (inc/fmha_i8.cuh:327-328) is taken on the sum, between magic - 127 and magic + 127
      for (int bb = 0; bb < 4; ++bb)
        y[bb] = __builtin_amdgcn_fmed3f(__builtin_fmaf(FASTACC ? o_f[u][4 * a + bb] + corr : o_f[u][4 * a + bb], fin, magic),
                                        magic_lo, magic_hi);
      const int lo = __builtin_amdgcn_perm(__float_as_int(y[1]), __float_as_int(y[0]), 0x0c0c0400);
      const int hi = __builtin_amdgcn_perm(__float_as_int(y[3]), __float_as_int(y[2]), 0x0c0c0400);
      w[u][a] = __builtin_amdgcn_perm(hi, lo, 0x05040100);
    }
  // Lanes l and l+32 hold the g = 0 / g = 1 words of the same query row.  One v_permlane32_swap per word hands lane l
  // both words of output tile u and lane l+32 both words of tile u+1: every lane then owns 32 contiguous bytes of a
  // row and writes them with two 128-bit stores instead of eight scattered 32-bit ones.
  if (row0 + i32 >= Sq) return;  // (no barrier follows)
  if (!fmha_in_bounds(row0 + i32 >= 0 && q_head_off + (long)(row0 + i32 + 1) * D <= (long)args.total_wgs / args.q_blocks * Sq * D))
    return;
  int8_t* op = args.o + q_head_off + (long)(row0 + i32) * D + 32 * g;
#pragma unroll
  for (int u = 0; u < kDSteps; u += 2) {
    int g0[4], g1[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const auto r = __builtin_amdgcn_permlane32_swap(w[u][a], w[u + 1][a], false, false);
      g0[a] = r[0];
      g1[a] = r[1];
    }
    *reinterpret_cast<v4i*>(op + 32 * u) = v4i{g0[0], g1[0], g0[1], g1[1]};
    *reinterpret_cast<v4i*>(op + 32 * u + 16) = v4i{g0[2], g1[2], g0[3], g1[3]};
  }
}

}  // namespace fmha_i8_gfx950
