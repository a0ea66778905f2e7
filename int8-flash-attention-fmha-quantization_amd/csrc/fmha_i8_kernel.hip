// INT8 fused multi-head flash attention for gfx950 (MI355X, CDNA4).  One kernel, templated on head_dim.
//
// What it computes is what the reference's FMHAInferKernel computes (inc/fmha_i8.cuh:43-334): per (batch, head),
// S = Q.K^T in int32, dequantised by 1/sqrt(d) * q_amax*k_amax/127^2, softmax over blocks of 128 keys against the
// BLOCK-LOCAL row maximum, P requantised to int8 in [-128,0] (scale -128, round-half-even), O~ = P.V in int32,
// online (m, l, O) merge across key blocks, and O requantised to int8 with v_amax/(128*o_amax), clamp +-127.
//
// How it computes it is designed for CDNA4, not taken from the reference:
//   * grid over (query block of 128 rows) x head x batch, XCD-aware so that the query blocks of one head share an L2;
//     4 wavefronts of 64 lanes per workgroup, each wavefront owns 32 query rows;
//   * both GEMMs run on v_mfma_i32_32x32x32_i8 in the TRANSPOSED formulation S^T = K.Q^T and O^T = V^T.P^T: each
//     lane then owns one query column, so the row max / row sum are in-register reductions plus one exchange with
//     lane^32, and the quantised P^T tile leaves the accumulator already in the B-operand register layout;
//   * K and V tiles of 128 keys are staged in LDS as [key][d] with the 16-byte chunk index XOR-swizzled by the row,
//     so that the 128-bit operand reads of K and the transposing reads of V (ds_read_b64_tr_b8) are bank-conflict
//     free; HBM is read with coalesced 128-bit loads, Q once per workgroup straight into MFMA operand registers;
//   * exp runs in the base-2 domain with all scales folded into one fma; P is converted to int8 with a
//     magic-number fma and packed with byte permutes; O is normalised once, in the epilogue.
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

__device__ __forceinline__ int pack4_low_bytes(float y0, float y1, float y2, float y3) {
  // the low byte of each magic-biased float is the two's-complement int8
  const int lo = __builtin_amdgcn_perm(__float_as_int(y1), __float_as_int(y0), 0x0c0c0400);
  const int hi = __builtin_amdgcn_perm(__float_as_int(y3), __float_as_int(y2), 0x0c0c0400);
  return __builtin_amdgcn_perm(hi, lo, 0x05040100);
}

template <int D>
__global__ __launch_bounds__(kThreads, 2) void fmha_i8_fwd_kernel(const KernelArgs args) {
  constexpr int kChunks = D / 16;                     // 16-byte chunks per row
  constexpr int kTileBytes = kBlockK * D;             // one K or V tile
  constexpr int kLoadsPerThread = kTileBytes / 16 / kThreads;
  constexpr int kDSteps = D / 32;                     // MFMA k-steps of GEMM 1, and 32-row output tiles of GEMM 2
  constexpr int kKeyTiles = kBlockK / 32;

  __shared__ __attribute__((aligned(16))) int8_t lds[2 * kTileBytes];
  __shared__ int lds_last_block;
  int8_t* const lds_k = lds;
  int8_t* const lds_v = lds + kTileBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
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

  // ---- last key block that holds any unmasked key (trailing padding is never loaded) -------------------------
  if (tid == 0) lds_last_block = -1;
  __syncthreads();
  for (int blk = tid; blk < n_blocks; blk += kThreads) {
    const int8_t* mp = mg + blk * kBlockK;
    bool valid = false;
    for (int j = 0; j < kBlockK; ++j) valid |= (mp[j] == 0);
    if (valid) atomicMax(&lds_last_block, blk);
  }

  // ---- Q: B operand of GEMM 1, loaded once -----------------------------------------------------------------------
  v4i qreg[kDSteps];
  {
    const int8_t* qp = args.q + head_off + (long)(qb * kBlockQ + wave * 32 + i32) * D + 16 * g;
#pragma unroll
    for (int kk = 0; kk < kDSteps; ++kk) qreg[kk] = *reinterpret_cast<const v4i*>(qp + 32 * kk);
  }
  __syncthreads();
  const int kb_end = lds_last_block + 1;

  // ---- per-lane LDS addressing -----------------------------------------------------------------------------------
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
  int st_off_k[kLoadsPerThread], st_off_v[kLoadsPerThread], ld_off[kLoadsPerThread];
#pragma unroll
  for (int it = 0; it < kLoadsPerThread; ++it) {
    const int ci = tid + kThreads * it;
    const int row = ci / kChunks, c = ci % kChunks;
    ld_off[it] = ci * 16;
    st_off_k[it] = row * D + ((c ^ k_swizzle<D>(row)) << 4);
    st_off_v[it] = row * D + ((c ^ v_swizzle<D>(row)) << 4);
  }

  float o_f[kDSteps][16];
#pragma unroll
  for (int u = 0; u < kDSteps; ++u)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_f[u][r] = 0.f;
  float m_run = args.floor2;  // running row maximum, base-2 units (inc/fmha_i8.cuh:91)
  float l_run = 0.f;          // running row sum (inc/fmha_i8.cuh:92)

  v4i pre_k[kLoadsPerThread], pre_v[kLoadsPerThread];
  int pre_mask = 0;
  auto prefetch = [&](int kb) {
    const int8_t* kp = kg + (long)kb * kTileBytes;
    const int8_t* vp = vg + (long)kb * kTileBytes;
#pragma unroll
    for (int it = 0; it < kLoadsPerThread; ++it) {
      pre_k[it] = *reinterpret_cast<const v4i*>(kp + ld_off[it]);
      pre_v[it] = *reinterpret_cast<const v4i*>(vp + ld_off[it]);
    }
    // 128 mask bytes of the block as 32 dwords in lanes 0..31 (assembled from bytes: the mask has no alignment rule)
    const int8_t* mp = mg + kb * kBlockK + 4 * i32;
    pre_mask = (mp[0] != 0 ? 1 : 0) | (mp[1] != 0 ? 2 : 0) | (mp[2] != 0 ? 4 : 0) | (mp[3] != 0 ? 8 : 0);
  };
  if (kb_end > 0) prefetch(0);

  for (int kb = 0; kb < kb_end; ++kb) {
    __syncthreads();  // every wave is done reading the previous tiles
#pragma unroll
    for (int it = 0; it < kLoadsPerThread; ++it) {
      *reinterpret_cast<v4i*>(lds_k + st_off_k[it]) = pre_k[it];
      *reinterpret_cast<v4i*>(lds_v + st_off_v[it]) = pre_v[it];
    }
    const int blk_mask = pre_mask;
    __syncthreads();
    if (kb + 1 < kb_end) prefetch(kb + 1);

    const unsigned long long any_masked = __ballot(blk_mask != 0);
    const unsigned long long all_masked = __ballot(blk_mask == 15);
    if (all_masked == ~0ull) continue;  // wave-uniform: nothing in this block is attended to

    // ---- GEMM 1: S^T[key][query] = K . Q^T, int32 (inc/fmha_i8.cuh:120-172) ---------------------------------------
    v16i acc[kKeyTiles];
#pragma unroll
    for (int t = 0; t < kKeyTiles; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0;
#pragma unroll
    for (int kk = 0; kk < kDSteps; ++kk)
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        const v4i a = *reinterpret_cast<const v4i*>(lds_k + k_read_off[kk] + 32 * t * D);
        acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, qreg[kk], acc[t], 0, 0, 0);
      }
    // lane holds, for query column i32, keys 32t + 8a + 4g + bb at acc[t][4a+bb]

    // ---- block softmax (inc/fmha_i8.cuh:174-253) -----------------------------------------------------------------
    v4i pk[kKeyTiles];
    float m_blk, l_blk = 0.f;
    if (any_masked == 0) {
      int top = acc[0][0];
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) top = max(top, acc[t][r]);
      top = max(top, __shfl_xor(top, 32));
      m_blk = fmaxf((float)top * args.c2, args.floor2);
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        float y[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf((float)acc[t][r], args.c2, -m_blk));
          l_blk += p;
          y[r] = __builtin_fmaf(p, -128.f, 12582912.f);  // 1.5*2^23 + rne(-128 p): low byte = int8 P
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) pk[t][a] = pack4_low_bytes(y[4 * a], y[4 * a + 1], y[4 * a + 2], y[4 * a + 3]);
      }
    } else {
      // some keys of this block are masked out (nonzero mask byte, inc/fmha_i8.cuh:189-192,216-221)
      unsigned mbits[kKeyTiles];  // bit 4a+bb of mbits[t] <-> key 32t + 8a + 4g + bb
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        unsigned bits = 0;
#pragma unroll
        for (int a = 0; a < 4; ++a) bits |= (unsigned)__shfl(blk_mask, 8 * t + 2 * a + g) << (4 * a);
        mbits[t] = bits;
      }
      float top = args.floor2;
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          top = fmaxf(top, ((mbits[t] >> r) & 1) ? args.masked2 : (float)acc[t][r] * args.c2);
      m_blk = fmaxf(top, __shfl_xor(top, 32));
#pragma unroll
      for (int t = 0; t < kKeyTiles; ++t) {
        float y[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float p = __builtin_amdgcn_exp2f(__builtin_fmaf((float)acc[t][r], args.c2, -m_blk));
          p = ((mbits[t] >> r) & 1) ? 0.f : p;
          l_blk += p;
          y[r] = __builtin_fmaf(fminf(p, 1.0f), -128.f, 12582912.f);
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) pk[t][a] = pack4_low_bytes(y[4 * a], y[4 * a + 1], y[4 * a + 2], y[4 * a + 3]);
      }
    }
    l_blk += __shfl_xor(l_blk, 32);

    // ---- GEMM 2: O~^T[d][query] = V^T . P^T, int32 (inc/fmha_i8.cuh:255-296) ---------------------------------------
    v16i oacc[kDSteps];
#pragma unroll
    for (int u = 0; u < kDSteps; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[u][r] = 0;
#pragma unroll
    for (int t = 0; t < kKeyTiles; ++t)
#pragma unroll
      for (int u = 0; u < kDSteps; ++u) {
        typedef v2i __attribute__((address_space(3))) * lds_v2i_ptr;
        const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(lds_v + v_read_off[u] + 32 * t * D));
        const v2i hi =
            __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_ptr)(lds_v + v_read_off[u] + 32 * t * D + 16 * D));
        const v4i a = {lo[0], lo[1], hi[0], hi[1]};
        oacc[u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, pk[t], oacc[u], 0, 0, 0);
      }
    // lane holds, for query column i32, output dims 32u + 8a + 4g + bb at oacc[u][4a+bb]

    // ---- online merge, normalisation deferred to the epilogue (inc/fmha_i8.cuh:298-315) ---------------------------
    const float m_new = fmaxf(m_run, m_blk);
    const float keep = __builtin_amdgcn_exp2f(m_run - m_new);
    const float take = __builtin_amdgcn_exp2f(m_blk - m_new);
    l_run = keep * l_run + take * l_blk;
    m_run = m_new;
    const float neg_take = -take;  // P carries the sign: P = -128 p (inc/fmha_i8.cuh:298)
#pragma unroll
    for (int u = 0; u < kDSteps; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r) o_f[u][r] = __builtin_fmaf(neg_take, (float)oacc[u][r], keep * o_f[u][r]);
  }

  // ---- epilogue: normalise, requantise, store (inc/fmha_i8.cuh:318-332) --------------------------------------------
  const float fin = (l_run > 0.f) ? args.out_scale / l_run : 0.f;  // a row with no unmasked key yields 0
  int8_t* op = args.o + head_off + (long)(qb * kBlockQ + wave * 32 + i32) * D + 4 * g;
#pragma unroll
  for (int u = 0; u < kDSteps; ++u)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      float y[4];
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        const float val = fminf(fmaxf(o_f[u][4 * a + bb] * fin, -127.f), 127.f);
        y[bb] = val + 12582912.f;  // round-half-even into the low mantissa byte
      }
      *reinterpret_cast<int*>(op + 32 * u + 8 * a) = pack4_low_bytes(y[0], y[1], y[2], y[3]);
    }
}

}  // namespace fmha_i8_gfx950
