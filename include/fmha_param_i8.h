/*
 * Parameter blocks of the INT8 fused multi-head attention launch API.
 *
 * Both structs are passed BY VALUE across the C ABI, so their field order, types and sizes are part of
 * the contract.  They restate the two PODs of the reference (inc/fmha_param_i8.h:3-8 AttnDataDescriptor,
 * inc/fmha_param_i8.h:10-17 FMHAParamI8): same field order, same types, same defaults.
 */
#ifndef FMHA_PARAM_I8_H_
#define FMHA_PARAM_I8_H_

#ifdef __cplusplus
#define FMHA_I8_DEFAULT(v) = v
#else
#define FMHA_I8_DEFAULT(v)
#endif

/* Shape of one attention call.  Q, K, V and O are int8 [batch_num, head_num, seq_len, head_dim], row-major and
 * contiguous; padding_mask is int8 [batch_num, seq_len] over KEY positions (reference: inc/fmha_param_i8.h:3-8). */
typedef struct AttnDataDescriptor {
  int batch_num FMHA_I8_DEFAULT(1);
  int seq_len FMHA_I8_DEFAULT(64);
  int head_num FMHA_I8_DEFAULT(4);
  int head_dim FMHA_I8_DEFAULT(64);
} AttnDataDescriptor;

/* Per-tensor symmetric quantization scales: x_fp32 ~= x_int8 * amax / 127 (reference: inc/fmha_param_i8.h:10-17).
 * s_max is carried for layout compatibility; neither the reference kernel nor this one reads it. */
typedef struct FMHAParamI8 {
  float q_amax FMHA_I8_DEFAULT(0.0f);
  float k_amax FMHA_I8_DEFAULT(0.0f);
  float v_amax FMHA_I8_DEFAULT(0.0f);
  float o_amax FMHA_I8_DEFAULT(1.0f);
  float s_max FMHA_I8_DEFAULT(1.0f);
} FMHAParamI8;

#undef FMHA_I8_DEFAULT

#ifdef __cplusplus
static_assert(sizeof(AttnDataDescriptor) == 16, "AttnDataDescriptor is 4 x int");
static_assert(sizeof(FMHAParamI8) == 20, "FMHAParamI8 is 5 x float");
#endif

#endif /* FMHA_PARAM_I8_H_ */
