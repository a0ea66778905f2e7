// INT8 fused multi-head flash attention for gfx950 (MI355X, CDNA4).  One kernel, templated on head_dim.
//
// What it computes is what the reference's FMHAInferKernel computes (inc/fmha_i8.cuh:43-334): per (batch, head),
// S = Q.K^T in int32, dequantised by 1/sqrt(d) * q_amax*k_amax/127^2, softmax over blocks of 128 keys against the
// BLOCK-LOCAL row maximum, P requantised to int8 in [-128,0] (scale -128, round-half-even), O~ = P.V in int32,
// online (m, l, O) merge across key blocks, and O requantised to int8 with v_amax/(128*o_amax), clamp +-127.
//
// How it computes it is designed for CDNA4, not taken from the reference:
//   * grid over (query block of 128 rows) x head x batch, XCD-aware so that the query blocks of one head share an L2;
//     4 wavefronts of 64 lanes per workgroup, each wavefront owns 32 query rows; 2 workgroups per CU;
//   * both GEMMs run on v_mfma_i32_32x32x32_i8 in the TRANSPOSED formulation S^T = K.Q^T and O^T = V^T.P^T: each
//     lane then owns one query column, so the row max / row sum are in-register reductions plus one exchange with
//     lane^32, and the quantised P^T tile leaves the accumulator already in the B-operand register layout;
//   * K and V tiles of 128 keys go HBM -> LDS directly (global_load_lds_dwordx4, no VGPR staging, no ds_write),
//     double buffered, as [key][d] with the 16-byte chunk index XOR-swizzled by the row (the swizzle is applied to the
//     global address each lane fetches), so that the 128-bit operand reads of K and the transposing reads of V
//     (ds_read_b64_tr_b8) are bank-conflict free; Q goes once per workgroup straight into MFMA operand registers;
//   * the softmax is written for the VALU issue port, which is what bounds this kernel: exp in the base-2 domain
//     with every scale folded into one fma, v_max3 for the row maximum, P converted AND packed by one SDWA subtract
//     per element (magic-number rounding, result byte written in place), the int32 accumulators of both GEMMs start
//     at the bit pattern of 1.5*2^23 so that they can be read as floats without a convert, the running O is only
//     rescaled when a row maximum jumps by more than 2^kLazyLog2, and O is normalised once, in the epilogue.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fmha_i8_gfx950 {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBlockQ = 128;   // query rows per workgroup
constexpr int kBlockK = 128;   // keys per softmax block (the reference's BASE_SEQ_LEN, src/fmha_i8.cu:61-95)
constexpr int kThreads = 256;  // 4 wavefronts
constexpr int kXcds = 8;
constexpr int kMaxKeyBlocks = 512;       // seq_len <= 65536
constexpr float kMagic = 12582912.0f;    // 1.5 * 2^23: float whose low mantissa bits hold a small signed integer
constexpr int kMagicBits = 0x4B400000;   // its bit pattern; kMagicBits + n is the float kMagic + n for |n| < 2^22
constexpr float kBiasOffsetLimit = 4096.0f;  // see the launch code: bound on the exponent offset of the biased path
constexpr float kLog2Pscale = -7.99995597f;  // log2(128 / 32767): exp2(x + kLog2Pscale) = 128 p / 32767
constexpr float kLazyLog2 = 10.0f;       // the running O is rescaled only when a row maximum grows by more than this

struct KernelArgs {
  const int8_t* q;
  const int8_t* k;
  const int8_t* v;
  const int8_t* mask;
  int8_t* o;
  int seq_len;
  int head_num;
  int q_blocks;     // seq_len / kBlockQ
  int total_wgs;    // batch * head_num * q_blocks
  float c2;         // log2(e) * (1/sqrt(d)) * q_amax*k_amax/127^2 : int32 S -> base-2 exponent
  float floor2;     // log2(e) * -1e6 : the reference's initial block maximum (inc/fmha_i8.cuh:116)
  float masked2;    // c2 * -1000000 : what a masked key contributes to the block maximum (inc/fmha_i8.cuh:191-193)
  float out_scale;  // v_amax / (o_amax * 128)   (inc/fmha_i8.cuh:318)
};

// 16-byte-chunk swizzles.  K is read 32 consecutive rows at a time (ds_read_b128); V is read by ds_read_b64_tr_b8
// whose 16-lane groups touch keys {0,1,2,3,8,9,10,11} (+4, +16, +20) of a 32-key slab.
template <int D>
__device__ __forceinline__ int k_swizzle(int row) {
  return D == 128 ? (row & 7) : ((row >> 1) & 3);
}
template <int D>
__device__ __forceinline__ int v_swizzle(int key) {
  return D == 128 ? ((key & 3) | ((key >> 1) & 4)) : (((key >> 1) & 1) | ((key >> 2) & 2));
}

// Four floats y_i in [-1, 1] -> four int8 bytes rne(32767 * y_i), packed in order.  v_cvt_pknorm_i16_f32 converts two at a
// time (round to nearest; exact .5 ties toward zero, which real softmax values do not hit), v_perm_b32 keeps the low
// byte of each 16-bit result.
typedef short v2s __attribute__((ext_vector_type(2)));
__device__ __forceinline__ int pack4_snorm(float y0, float y1, float y2, float y3) {
  const v2s lo = __builtin_amdgcn_cvt_pknorm_i16(y0, y1);
  const v2s hi = __builtin_amdgcn_cvt_pknorm_i16(y2, y3);
  return __builtin_amdgcn_perm(__builtin_bit_cast(int, hi), __builtin_bit_cast(int, lo), 0x06040200);
}
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

// BIAS: the S accumulators start at kMagicBits and are read as floats (no int->float convert).  Exact only while
// (kMagic + |S|) * c2 stays small enough for the float grid; the host selects it from c2.
template <int D, bool BIAS>
__global__ __launch_bounds__(kThreads, 2) void fmha_i8_fwd_kernel(const KernelArgs args) {
  constexpr int kChunks = D / 16;                     // 16-byte chunks per row
  constexpr int kTileBytes = kBlockK * D;             // one K or V tile
  constexpr int kRegionsPerWave = kTileBytes / 1024 / 4;  // 1 KiB (64 lanes x 16 B) direct-to-LDS loads per wave
  constexpr int kRowsPerRegion = 1024 / D;
  constexpr int kDSteps = D / 32;                     // MFMA k-steps of GEMM 1, and 32-row output tiles of GEMM 2
  constexpr int kKeyTiles = kBlockK / 32;

  __shared__ __attribute__((aligned(1024))) int8_t lds[2][2][kTileBytes];  // [buffer][K|V][tile]
  __shared__ unsigned char lds_class[kMaxKeyBlocks];  // per key block: bit0 = some key masked, bit1 = all keys masked
  __shared__ int lds_last_block;

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
  const int S = args.seq_len;
  const long head_off = (long)bh * S * D;
  const int8_t* __restrict__ kg = args.k + head_off;
  const int8_t* __restrict__ vg = args.v + head_off;
  const int8_t* __restrict__ mg = args.mask + (long)b * S;
  const int n_blocks = S / kBlockK;

  // ---- classify the key blocks of this batch entry: 4 mask bytes per lane, two blocks per wavefront ballot ---------
  if (tid == 0) lds_last_block = -1;
  __syncthreads();
  for (int base = 0; base < S; base += 4 * kThreads) {
    const int j = base + 4 * tid;
    int nib = 15;
    if (j < S) nib = (mg[j] != 0 ? 1 : 0) | (mg[j + 1] != 0 ? 2 : 0) | (mg[j + 2] != 0 ? 4 : 0) | (mg[j + 3] != 0 ? 8 : 0);
    const unsigned long long some = __ballot(nib != 0), all = __ballot(nib == 15);
    if ((lane & 31) == 0 && j < S) {
      const unsigned half_some = (unsigned)(some >> (lane & 32)), half_all = (unsigned)(all >> (lane & 32));
      const int blk = j / kBlockK;
      const int cls = (half_some != 0 ? 1 : 0) | (half_all == 0xffffffffu ? 2 : 0);
      lds_class[blk] = (unsigned char)cls;
      if (!(cls & 2)) atomicMax(&lds_last_block, blk);
    }
  }

  // ---- Q: B operand of GEMM 1, loaded once -----------------------------------------------------------------------
  v4i qreg[kDSteps];
  {
    const int8_t* qp = args.q + head_off + (long)(qb * kBlockQ + wave * 32 + i32) * D + 16 * g;
#pragma unroll
    for (int kk = 0; kk < kDSteps; ++kk) qreg[kk] = *reinterpret_cast<const v4i*>(qp + 32 * kk);
  }
  __syncthreads();
  const int kb_end = __builtin_amdgcn_readfirstlane(lds_last_block) + 1;

  // ---- per-lane addressing -----------------------------------------------------------------------------------------
  // direct-to-LDS loads: lane l of a 1 KiB region lands at byte 16*l of the region, so the lane FETCHES the chunk that
  // the swizzle assigns to that slot.
  int ld_goff_k, ld_goff_v;
  {
    const int row_in = lane / kChunks, p = lane % kChunks;
    const int vrow = (D == 128) ? (row_in | ((wave & 1) << 3)) : row_in;  // row bits the V swizzle looks at
    ld_goff_k = row_in * D + ((p ^ k_swizzle<D>(row_in)) << 4);
    ld_goff_v = row_in * D + ((p ^ v_swizzle<D>(vrow)) << 4);
  }
  int k_read_off[kDSteps];  // + 32*t*D per key tile
#pragma unroll
  for (int kk = 0; kk < kDSteps; ++kk)
    k_read_off[kk] = i32 * D + (((2 * kk + g) ^ k_swizzle<D>(i32)) << 4);
  int v_read_off[kDSteps];  // + 32*t*D per key tile, + 16*D for the second half of the operand
  {
    const int jin = lane & 15, hh = (lane >> 4) & 1;
    const int kslot = jin >> 1;
    const int key_lane = 4 * g + (kslot < 4 ? kslot : kslot + 4);
#pragma unroll
    for (int u = 0; u < kDSteps; ++u)
      v_read_off[u] = key_lane * D + (((2 * u + hh) ^ v_swizzle<D>(key_lane)) << 4) + 8 * (jin & 1);
  }

  // HBM -> LDS without passing through registers.  Written as inline assembly on purpose: the compiler treats an
  // LDS-DMA builtin as a store that may alias every later LDS read and would wait for the NEXT tile (vmcnt(0)) before
  // the first operand read of the CURRENT one.  Completion is tracked by hand: s_waitcnt vmcnt(0) + barrier at the top
  // of each iteration.  M0 carries the LDS destination of lane 0; lane l lands 16*l bytes further.
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int8_t*)&lds[0][0][0];
  auto issue_tile_loads = [&](int kb, int buf) {
    const int8_t* kp = kg + (long)kb * kTileBytes;  // wave-uniform bases (SGPR pairs)
    const int8_t* vp = vg + (long)kb * kTileBytes;
#pragma unroll
    for (int it = 0; it < kRegionsPerWave; ++it) {
      const int region = it * 4 + wave;
      const unsigned dst_k = lds_base + (unsigned)((buf * 2 + 0) * kTileBytes + region * 1024);
      const unsigned dst_v = lds_base + (unsigned)((buf * 2 + 1) * kTileBytes + region * 1024);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :: "s"(dst_k), "v"(ld_goff_k + region * 1024), "s"(kp) : "memory");
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                   :: "s"(dst_v), "v"(ld_goff_v + region * 1024), "s"(vp) : "memory");
    }
  };

  float o_f[kDSteps][16];
#pragma unroll
  for (int u = 0; u < kDSteps; ++u)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_f[u][r] = 0.f;
  float m_ref = args.floor2 - 2.f * kLazyLog2;  // reference exponent of the running O and l (base-2 units)
  float l_run = 0.f;                            // running row sum, in units of 1/128 (it sums 128*p)
  const float c2 = args.c2;
  const float bias_c2 = BIAS ? kMagic * c2 : 0.f;
  const float magic = kMagic;
  v16i magic_c;  // C operand that starts an accumulation chain at kMagicBits without per-element moves
#pragma unroll
  for (int r = 0; r < 16; ++r) magic_c[r] = kMagicBits;
  asm volatile("" : "+v"(magic_c));  // keep it in registers: 16 moves once, not 128 per key block

  // Make the compiler retire its own outstanding loads (Q) here: its later vmcnt bookkeeping does not know about the
  // hand-issued LDS-DMA loads and would otherwise wait for them inside the loop.
#pragma unroll
  for (int kk = 0; kk < kDSteps; ++kk) asm volatile("" ::"v"(qreg[kk]));
  if (kb_end > 0) issue_tile_loads(0, 0);

  for (int kb = 0; kb < kb_end; ++kb) {
    const int buf = kb & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // tile kb has landed for every wave; every wave is done reading the other buffer
    if (kb + 1 < kb_end) issue_tile_loads(kb + 1, buf ^ 1);
    const int cls = __builtin_amdgcn_readfirstlane((int)lds_class[kb]);
    if (cls & 2) continue;  // nothing in this block is attended to
    const int8_t* lds_k = &lds[buf][0][0];
    const int8_t* lds_v = &lds[buf][1][0];

    // ---- GEMM 1: S^T[key][query] = K . Q^T, int32 (inc/fmha_i8.cuh:120-172) ---------------------------------------
    v16i acc[kKeyTiles];
    const v16i zero_c = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    {
      // operand reads run one k-step ahead of the MFMAs that consume them
      v4i ka[2][kKeyTiles];
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) ka[0][t] = *reinterpret_cast<const v4i*>(lds_k + k_read_off[0] + 32 * t * D);
#pragma unroll
      for (int kk = 0; kk < kDSteps; ++kk) {
        if (kk + 1 < kDSteps) {
#pragma unroll
          for (int t = 0; t < kKeyTiles; ++t)
            ka[(kk + 1) & 1][t] = *reinterpret_cast<const v4i*>(lds_k + k_read_off[kk + 1] + 32 * t * D);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < kKeyTiles; ++t)
          acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka[kk & 1][t], qreg[kk],
                                                         kk == 0 ? (BIAS ? magic_c : zero_c) : acc[t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // lane holds, for query column i32, keys 32t + 8a + 4g + bb at acc[t][4a+bb]

    // ---- block softmax (inc/fmha_i8.cuh:174-253) -----------------------------------------------------------------
    // sf(t,r): the score as a float; with BIAS it still carries +kMagic, which the exponent offset removes.
    auto sf = [&](int t, int r) -> float { return BIAS ? __int_as_float(acc[t][r]) : (float)acc[t][r]; };
    v4i pk[kKeyTiles];
    float m_blk;        // block-local row maximum, base-2 units
    float l_blk = 0.f;  // sum of 128*p over this lane's keys
    if (cls == 0) {
      // integer maximum (monotone in the score, also for the biased bit patterns), two independent chains
      constexpr int kVals = 16 * kKeyTiles;  // scores per lane; v(n) = acc[n / 16][n % 16]
      int t0 = acc[0][0], t1 = acc[0][1];
#pragma unroll
      for (int n = 2; n + 3 < kVals; n += 4) {
        t0 = max(max(t0, acc[n / 16][n % 16]), acc[(n + 1) / 16][(n + 1) % 16]);
        t1 = max(max(t1, acc[(n + 2) / 16][(n + 2) % 16]), acc[(n + 3) / 16][(n + 3) % 16]);
      }
      t0 = max(max(t0, acc[kKeyTiles - 1][14]), acc[kKeyTiles - 1][15]);
      const int ti = half_max(max(t0, t1));
      const float top = BIAS ? __int_as_float(ti) : (float)ti;
      // off = top*c2 rounded; p' = exp2(s*c2 - off) = p * 2^(resid) with one row-wide resid below 1 ulp of off, and the
      // block maximum that is consistent with p' is off itself (minus the constant kMagic*c2 when BIAS).
      float off = top * c2;
      if (!BIAS) off = fmaxf(off, args.floor2);
      m_blk = off - bias_c2;
      const float offq = off - kLog2Pscale;  // exp2(x - offq) = 128 p / 32767: the snorm conversion returns rne(128 p)
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sf(t, 4 * a + 0), c2, -offq));
          const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sf(t, 4 * a + 1), c2, -offq));
          const float e2 = __builtin_amdgcn_exp2f(__builtin_fmaf(sf(t, 4 * a + 2), c2, -offq));
          const float e3 = __builtin_amdgcn_exp2f(__builtin_fmaf(sf(t, 4 * a + 3), c2, -offq));
          l_blk += (e0 + e1) + (e2 + e3);
          pk[t][a] = pack4_snorm(-e0, -e1, -e2, -e3);
        }
    } else {
      // some keys of this block are masked out (nonzero mask byte, inc/fmha_i8.cuh:189-192,216-221)
      const int8_t* mp = mg + kb * kBlockK + 4 * i32;
      const int nib = (mp[0] != 0 ? 1 : 0) | (mp[1] != 0 ? 2 : 0) | (mp[2] != 0 ? 4 : 0) | (mp[3] != 0 ? 8 : 0);
      unsigned mbits[kKeyTiles];  // bit 4a+bb of mbits[t] <-> key 32t + 8a + 4g + bb
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        unsigned bits = 0;
#pragma unroll
        for (int a = 0; a < 4; ++a) bits |= (unsigned)__shfl(nib, 8 * t + 2 * a + g) << (4 * a);
        mbits[t] = bits;
      }
      const float masked_s = args.masked2 + bias_c2;  // in the units of sf()*c2
      float top = args.floor2 + bias_c2;
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) top = fmaxf(top, ((mbits[t] >> r) & 1) ? masked_s : sf(t, r) * c2);
      const float off = half_max(top);
      m_blk = off - bias_c2;
      const float offq = off - kLog2Pscale;
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          float e[4];
#pragma unroll
          for (int bb = 0; bb < 4; ++bb) {
            const int r = 4 * a + bb;
            const float ex = __builtin_amdgcn_exp2f(__builtin_fmaf(sf(t, r), c2, -offq));
            e[bb] = ((mbits[t] >> r) & 1) ? 0.f : ex;
            l_blk += e[bb];
          }
          pk[t][a] = pack4_snorm(-e[0], -e[1], -e[2], -e[3]);
        }
    }
    l_blk = half_sum(l_blk);

    // ---- GEMM 2: O~^T[d][query] = V^T . P^T, int32 (inc/fmha_i8.cuh:255-296); accumulators start at kMagicBits ----
    v16i oacc[kDSteps];
    {
      typedef v2i __attribute__((address_space(3))) * lds_v2i_ptr;
      v2i va[2][kDSteps][2];  // transposed V operands, one 32-key tile ahead of the MFMAs
#pragma unroll
      for (int u = 0; u < kDSteps; ++u) {
        va[0][u][0] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(lds_v + v_read_off[u]));
        va[0][u][1] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(lds_v + v_read_off[u] + 16 * D));
      }
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        if (t + 1 < kKeyTiles) {
#pragma unroll
          for (int u = 0; u < kDSteps; ++u) {
            va[(t + 1) & 1][u][0] =
                __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(lds_v + v_read_off[u] + 32 * (t + 1) * D));
            va[(t + 1) & 1][u][1] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                (lds_v2i_ptr)(lds_v + v_read_off[u] + 32 * (t + 1) * D + 16 * D));
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < kDSteps; ++u) {
          const v4i a = {va[t & 1][u][0][0], va[t & 1][u][0][1], va[t & 1][u][1][0], va[t & 1][u][1][1]};
          oacc[u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, pk[t], t == 0 ? magic_c : oacc[u], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // lane holds, for query column i32, output dims 32u + 8a + 4g + bb at oacc[u][4a+bb], as the float kMagic + O~

    // ---- online merge, normalisation deferred to the epilogue (inc/fmha_i8.cuh:298-315) ---------------------------
    // O and l are kept relative to 2^m_ref; m_ref only moves when some row's block maximum exceeds it by 2^kLazyLog2.
    if (__ballot(m_blk > m_ref + kLazyLog2) != 0) {
      const float m_new = fmaxf(m_ref, m_blk);
      const float keep = __builtin_amdgcn_exp2f(m_ref - m_new);
      m_ref = m_new;
      l_run *= keep;
#pragma unroll
      for (int u = 0; u < kDSteps; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_f[u][r] *= keep;
    }
    const float take = __builtin_amdgcn_exp2f(m_blk - m_ref);
    l_run = __builtin_fmaf(take, l_blk, l_run);
    const float neg_take = -take;  // P carries the sign: P = -128 p (inc/fmha_i8.cuh:298)
#pragma unroll
    for (int u = 0; u < kDSteps; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        o_f[u][r] = __builtin_fmaf(neg_take, __int_as_float(oacc[u][r]) - magic, o_f[u][r]);
  }

  // ---- epilogue: normalise, requantise, store (inc/fmha_i8.cuh:318-332) --------------------------------------------
  // l_run sums 128 p / 32767 and O sums 128 p v, so mean(v) = O / (32767 l_run); a row with no unmasked key yields 0
  const float fin = (l_run > 0.f) ? args.out_scale * (128.f / kSnorm) / l_run : 0.f;
  int8_t* op = args.o + head_off + (long)(qb * kBlockQ + wave * 32 + i32) * D + 4 * g;
#pragma unroll
  for (int u = 0; u < kDSteps; ++u)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      float y[4];
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) y[bb] = __builtin_amdgcn_fmed3f(o_f[u][4 * a + bb] * fin, -127.f, 127.f) + magic;
      // magic + y holds rne(y) in the low mantissa byte (round-half-even)
      const int lo = __builtin_amdgcn_perm(__float_as_int(y[1]), __float_as_int(y[0]), 0x0c0c0400);
      const int hi = __builtin_amdgcn_perm(__float_as_int(y[3]), __float_as_int(y[2]), 0x0c0c0400);
      *reinterpret_cast<int*>(op + 32 * u + 8 * a) = __builtin_amdgcn_perm(hi, lo, 0x05040100);
    }
}

}  // namespace fmha_i8_gfx950
