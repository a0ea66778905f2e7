// C ABI of libfmha_i8.so: argument checking, scale folding and the kernel launch.  Stands where the reference has
// FMHAInferI8 / LaunchFMHAInfer_TCU (src/fmha_i8.cu:31-173): the if/else ladder over (head_dim, seq_len) template
// instantiations becomes a run-time seq_len and a two-way switch on head_dim.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/fmha_i8.h"
#include "fmha_i8_kernel.hip"

namespace {

using fmha_i8_gfx950::KernelArgs;

// One shape for both entry points: self-attention is the case seq_len_q == seq_len_kv.
FMHACrossAttnDescriptor as_cross(const AttnDataDescriptor& a) {
  return FMHACrossAttnDescriptor{a.batch_num, a.seq_len, a.seq_len, a.head_num, a.head_dim};
}

// inc/fmha_i8.cuh:71-72: row_scale = 1/sqrt(d), scale_qk_out = q_amax*k_amax/127^2; folded with log2(e) because the
// kernel's exponentials are base 2.
float score_scale_log2(const FMHAParamI8& p, int head_dim) {
  constexpr float kLog2e = 1.4426950408889634f;
  const float row_scale = 1.0f / sqrtf((float)head_dim);
  const float scale_qk_out = p.q_amax * p.k_amax / (127.f * 127.f);
  return row_scale * scale_qk_out * kLog2e;
}
float output_scale(const FMHAParamI8& p) { return p.v_amax / (p.o_amax * 128.f); }  // inc/fmha_i8.cuh:318

int check_args(const FMHAParamI8& p, const FMHACrossAttnDescriptor& a, const void* q, const void* k, const void* v,
               const void* mask, const void* o) {
  if (!q || !k || !v || !mask || !o) return FMHA_I8_ERR_NULL_POINTER;
  if (a.head_dim != 64 && a.head_dim != 128) return FMHA_I8_ERR_HEAD_DIM;
  if (a.seq_len_kv <= 0 || a.seq_len_kv > 65536 || a.seq_len_q <= 0 || a.seq_len_q > 65536) return FMHA_I8_ERR_SEQ_LEN;
  if (a.batch_num <= 0 || a.head_num <= 0) return FMHA_I8_ERR_BATCH_HEAD;
  const long long wgs = (long long)a.batch_num * a.head_num * ((a.seq_len_q + fmha_i8_gfx950::kBlockQ - 1) / fmha_i8_gfx950::kBlockQ);
  if (wgs > 0x7fffffffLL) return FMHA_I8_ERR_BATCH_HEAD;
  const uintptr_t bits = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o;
  if (bits & 15u) return FMHA_I8_ERR_ALIGNMENT;
  if (!isfinite(p.q_amax) || !isfinite(p.k_amax) || !isfinite(p.v_amax) || !isfinite(p.o_amax) || !(p.o_amax > 0.f))
    return FMHA_I8_ERR_SCALE;
  // amax values are maxima of absolute values.  The kernel takes row maxima on the integer scores, which is only the
  // maximum of the scaled scores while the scale is not negative.
  if (p.q_amax * p.k_amax < 0.f) return FMHA_I8_ERR_SCALE;
  // Finite amax values can still overflow in the scales the kernel works with (1e20 * 1e20, 1e30 / 1e-30); an
  // infinite or NaN scale would turn every score or every output into NaN behind a status of "ok".
  if (!isfinite(score_scale_log2(p, a.head_dim)) || !isfinite(output_scale(p))) return FMHA_I8_ERR_SCALE;
  return FMHA_I8_OK;
}

struct Variant {
  bool bias, fast, full_range_p;
};
// Every launch hands back the status of THAT launch (the return value of hipLaunchKernel), never the thread's last
// error: an unrelated earlier failure of the caller must neither be reported as this call's nor be cleared by it.
template <int D, int BK, bool RAGGED, bool FULLP>
hipError_t launch_variant4(Variant var, dim3 grid, dim3 block, hipStream_t stream, const fmha_i8_gfx950::KernelArgs& args) {
  using namespace fmha_i8_gfx950;
  KernelArgs by_value = args;
  void* kernel_args[] = {&by_value};
#ifdef FMHA_FEW_INSTANTIATIONS
  // Test builds that are compiled many times over (tests/Makefile, target `variants`) carry only the instantiations
  // the five benchmark configurations use: blocks of 128 keys, whole blocks, 128-step P, the one-fma merge.
  if constexpr (BK != kBlockK || RAGGED || FULLP) return hipErrorInvalidDeviceFunction;
  else {
    if (!var.fast) return hipErrorInvalidDeviceFunction;
    return var.bias ? hipLaunchKernel(reinterpret_cast<const void*>(&fmha_i8_fwd_kernel<D, BK, true, true, RAGGED, FULLP>), grid, block, kernel_args, 0, stream)
                    : hipLaunchKernel(reinterpret_cast<const void*>(&fmha_i8_fwd_kernel<D, BK, false, true, RAGGED, FULLP>), grid, block, kernel_args, 0, stream);
  }
#else
#define FMHA_LAUNCH(BB, FF) \
  hipLaunchKernel(reinterpret_cast<const void*>(&fmha_i8_fwd_kernel<D, BK, BB, FF, RAGGED, FULLP>), grid, block, kernel_args, 0, stream)
  if (var.bias) return var.fast ? FMHA_LAUNCH(true, true) : FMHA_LAUNCH(true, false);
  return var.fast ? FMHA_LAUNCH(false, true) : FMHA_LAUNCH(false, false);
#undef FMHA_LAUNCH
#endif
}
template <int D, int BK, bool RAGGED>
hipError_t launch_variant3(Variant var, dim3 grid, dim3 block, hipStream_t stream, const fmha_i8_gfx950::KernelArgs& args) {
  if (var.full_range_p) return launch_variant4<D, BK, RAGGED, true>(var, grid, block, stream, args);
  return launch_variant4<D, BK, RAGGED, false>(var, grid, block, stream, args);
}
template <int D, int BK>
hipError_t launch_variant(Variant var, dim3 grid, dim3 block, hipStream_t stream, const fmha_i8_gfx950::KernelArgs& args) {
  if (args.seq_kv % BK != 0) return launch_variant3<D, BK, true>(var, grid, block, stream, args);
  return launch_variant3<D, BK, false>(var, grid, block, stream, args);
}

int launch(hipStream_t stream, const FMHAParamI8& p, const FMHACrossAttnDescriptor& a, const void* q, const void* k,
           const void* v, const void* mask, void* o, bool full_range_p = false) {
  const int st = check_args(p, a, q, k, v, mask, o);
  if (st != FMHA_I8_OK) return st;
  constexpr float kLog2e = 1.4426950408889634f;
  KernelArgs args;
  args.q = static_cast<const int8_t*>(q);
  args.k = static_cast<const int8_t*>(k);
  args.v = static_cast<const int8_t*>(v);
  args.mask = static_cast<const int8_t*>(mask);
  args.o = static_cast<int8_t*>(o);
  args.seq_q = a.seq_len_q;
  args.seq_kv = a.seq_len_kv;
  args.head_num = a.head_num;
  args.q_blocks = (a.seq_len_q + fmha_i8_gfx950::kBlockQ - 1) / fmha_i8_gfx950::kBlockQ;
  args.total_wgs = a.batch_num * a.head_num * args.q_blocks;
  args.c2 = score_scale_log2(p, a.head_dim);
  // A masked score is replaced by -inf before it is scaled (see the kernel): the scale must not be exactly 0.  With
  // 1e-30 every exponent is below 1e-23 in magnitude and the probabilities are the same floats as with 0.
  if (args.c2 < 1e-30f) args.c2 = 1e-30f;
  args.floor2 = -1e6f * kLog2e;
  args.out_scale = output_scale(p);
  const dim3 grid((unsigned)args.total_wgs), block(fmha_i8_gfx950::kThreads);
  // The accumulators of Q.K^T can be read as floats without a convert when they start at the bit pattern of a float;
  // the price is that the exponent offset (start value*2^26 + S)*c2 is then rounded on a coarser float grid.  Take that
  // path only while the offset stays below 2^12, i.e. while the rounding moves a whole row by less than 2^-13 in log2.
  // (The start value and the bound on |S| depend on the head size: see score_base_bits in the kernel source.)
  const float offset_ulps = a.head_dim == 64
                                ? fmha_i8_gfx950::score_base_ulps<64>() + fmha_i8_gfx950::score_range_ulps<64>()
                                : fmha_i8_gfx950::score_base_ulps<128>() + fmha_i8_gfx950::score_range_ulps<128>();
  const bool bias = offset_ulps * fabsf(args.c2) < fmha_i8_gfx950::kBiasOffsetLimit;
  // Folding the accumulator offset into the running O (see FASTACC in the kernel) costs a rounding of relative size
  // 2^-24 at magnitude kBase * sum(take) per key block; normalised by the row sum (>= sum(take)) and scaled to output
  // LSBs that is at most about 0.0034 * (v_amax/o_amax) * sqrt(key blocks).  Take it while that stays below 0.1 LSB.
  // Blocks of 128 keys, as the reference uses for its multiples of 128; its other lengths (64, 192, 320, 448:
  // src/fmha_i8.cu:41-60) run in blocks of 64 keys, and so does every other odd multiple of 64 here.
  // A key count that is not a multiple of 64 is treated as the next multiple of 64 whose last keys are masked out.
  const int kv_padded = (a.seq_len_kv + fmha_i8_gfx950::kBlockKSmall - 1) / fmha_i8_gfx950::kBlockKSmall * fmha_i8_gfx950::kBlockKSmall;
  const int block_keys = kv_padded % fmha_i8_gfx950::kBlockK == 0 ? fmha_i8_gfx950::kBlockK : fmha_i8_gfx950::kBlockKSmall;
  const float lsb_bound = 0.0034f * fabsf(p.v_amax / p.o_amax) * sqrtf((float)(kv_padded / block_keys));
  const bool fast = lsb_bound < 0.1f;
  const Variant var{bias, fast, full_range_p};
  hipError_t err;
  if (a.head_dim == 128) {
    if (block_keys == fmha_i8_gfx950::kBlockK) err = launch_variant<128, fmha_i8_gfx950::kBlockK>(var, grid, block, stream, args);
    else err = launch_variant<128, fmha_i8_gfx950::kBlockKSmall>(var, grid, block, stream, args);
  } else {
    if (block_keys == fmha_i8_gfx950::kBlockK) err = launch_variant<64, fmha_i8_gfx950::kBlockK>(var, grid, block, stream, args);
    else err = launch_variant<64, fmha_i8_gfx950::kBlockKSmall>(var, grid, block, stream, args);
  }
  return err == hipSuccess ? FMHA_I8_OK : FMHA_I8_ERR_HIP_BASE + (int)err;
}

}  // namespace

extern "C" {

int FMHAInferI8CheckArgs(FMHAParamI8 fmha_param, AttnDataDescriptor attn_desc, const void* q, const void* k,
                         const void* v, const void* padding_mask, const void* o) {
  return check_args(fmha_param, as_cross(attn_desc), q, k, v, padding_mask, o);
}

int FMHAInferI8Status(hipStream_t stream, FMHAParamI8 fmha_param, AttnDataDescriptor attn_desc, const void* q,
                      const void* k, const void* v, const void* padding_mask, void* o, bool /*use_tcu*/) {
  return launch(stream, fmha_param, as_cross(attn_desc), q, k, v, padding_mask, o);
}

int FMHAInferI8Cross(hipStream_t stream, FMHAParamI8 fmha_param, FMHACrossAttnDescriptor desc, const void* q,
                     const void* k, const void* v, const void* padding_mask, void* o) {
  return launch(stream, fmha_param, desc, q, k, v, padding_mask, o);
}

int FMHAInferI8CrossFullRangeP(hipStream_t stream, FMHAParamI8 fmha_param, FMHACrossAttnDescriptor desc, const void* q,
                               const void* k, const void* v, const void* padding_mask, void* o) {
  return launch(stream, fmha_param, desc, q, k, v, padding_mask, o, true);
}

int FMHAInferI8CrossCheckArgs(FMHAParamI8 fmha_param, FMHACrossAttnDescriptor desc, const void* q, const void* k,
                              const void* v, const void* padding_mask, const void* o) {
  return check_args(fmha_param, desc, q, k, v, padding_mask, o);
}

void FMHAInferI8(hipStream_t stream, FMHAParamI8 fmha_param, AttnDataDescriptor attn_desc, const void* q, const void* k,
                 const void* v, const void* padding_mask, void* o, bool /*use_tcu*/) {
  const int st = launch(stream, fmha_param, as_cross(attn_desc), q, k, v, padding_mask, o);
  if (st != FMHA_I8_OK)
    fprintf(stderr, "FMHAInferI8: nothing launched, o left untouched: %s (B=%d H=%d S=%d d=%d)\n",
            FMHAInferI8StatusString(st), attn_desc.batch_num, attn_desc.head_num, attn_desc.seq_len,
            attn_desc.head_dim);
}

const char* FMHAInferI8StatusString(int status) {
  switch (status) {
    case FMHA_I8_OK: return "ok";
    case FMHA_I8_ERR_NULL_POINTER: return "null pointer argument";
    case FMHA_I8_ERR_HEAD_DIM: return "head_dim must be 64 or 128";
    case FMHA_I8_ERR_SEQ_LEN: return "seq_len must be between 1 and 65536 (queries and keys alike)";
    case FMHA_I8_ERR_BATCH_HEAD: return "batch_num and head_num must be positive (and the grid must fit)";
    case FMHA_I8_ERR_ALIGNMENT: return "q, k, v and o must be 16-byte aligned";
    case FMHA_I8_ERR_SCALE: return "amax values must be finite, o_amax > 0, q_amax * k_amax >= 0, and the scales derived from them finite";
    default: break;
  }
  if (status >= FMHA_I8_ERR_HIP_BASE) return hipGetErrorString((hipError_t)(status - FMHA_I8_ERR_HIP_BASE));
  return "unknown status";
}

#ifdef FMHA_CHECK_BOUNDS
// Test build only: the number of global accesses that would have left their tensor since the last call of this
// function (synchronises the device; see the kernel source).
int FMHAInferI8DebugOutOfBounds(void) {
  int count = -1, zero = 0;
  if (hipDeviceSynchronize() != hipSuccess) return -1;
  if (hipMemcpyFromSymbol(&count, HIP_SYMBOL(fmha_i8_gfx950::g_fmha_oob_count), sizeof(int)) != hipSuccess) return -1;
  if (hipMemcpyToSymbol(HIP_SYMBOL(fmha_i8_gfx950::g_fmha_oob_count), &zero, sizeof(int)) != hipSuccess) return -1;
  return count;
}
#endif

#ifdef FMHA_TRACE_TICKS
// Test build only: copies the first `words` time stamps of the last launch (see the kernel source) to host memory.
int FMHAInferI8DebugReadTrace(unsigned* dst, int words) {
  if (hipDeviceSynchronize() != hipSuccess) return -1;
  if (words < 0 || words > fmha_i8_gfx950::kTraceWorkgroups * 8 * 64) return -1;
  return hipMemcpyFromSymbol(dst, HIP_SYMBOL(fmha_i8_gfx950::g_fmha_trace), sizeof(unsigned) * words) == hipSuccess ? 0 : -1;
}
#endif

const char* FMHAInferI8Version(void) { return "fmha_i8 gfx950 mfma32x32x32 direct-to-lds two-phase"; }

}  // extern "C"
