/*
 * lf_attn_params.h — the parameter block of the attention kernels, for C and C++
 * hosts that launch them through lf_shim.h without Python.
 *
 * A kernel takes ONE argument, this struct by value; lf_launch receives
 * `void* args[1] = { &params }`.  It is the device-side `struct LfAttnParams`
 * (loopfuse_amd/csrc/kernels/lf_common.hip.h) restated with fixed-width host
 * types, field for field; loopfuse_amd/lowering.py::AttnParams is the ctypes
 * mirror.  It replaces the positional argument list of the reference's generated
 * launch function — tensors, then one stride per dimension, then the dimensions
 * (reference loopfuse/codegen.py:215-298, :241-242 for the strides).
 *
 * Strides are in ELEMENTS (bf16/fp16), the innermost dimension (head dim) has
 * stride 1 everywhere.  Pointers are device pointers, 16-byte aligned.
 */
#ifndef LF_ATTN_PARAMS_H
#define LF_ATTN_PARAMS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct LfAttnParamsHost {
  const void* q;        /* Q [B, Hq, Sq, D] */
  const void* k;        /* K [B, Hkv, Sk, D], or the K page pool when the kernel is built with LF_PAGED & 1 */
  const void* v;        /* V likewise (LF_PAGED & 2) */
  void* o;              /* O [B, Hq, Sq, D] */
  const void* k_table;  /* [B, pages] page ids, int32 or int64 (LF_TABLE_I64) */
  const void* v_table;
  float* part_acc;      /* decode split-K scratch: [units, nsplit, rows, D] floats; lf_attn_prefill_swp -DLF_BIAS=1 and
                           lf_bias_classify: int32 [units', kv tiles of 64] tile classes of the score bias (written by
                           lf_bias_classify, launched first with the same block; units' = distinct (batch, head) of the
                           bias x q tiles of the attention kernel) */
  float* part_ml;       /* decode split-K scratch: [units, nsplit, rows, 2] floats; lf_attn_prefill_swp: optional
                           output [B, Hq, Sq] floats, the rows' log-sum-exp in log2 units (NULL: not written) */
  unsigned char* visits;/* optional [B*Hq*q_tiles, kv_tiles] visited-tile record, else NULL */
  const void* bias;     /* LF_BIAS & 1: additive score bias [B, Hq, Sq, Sk]; lf_attn_decode -DLF_BIAS=1: [B, Hkv, rows, Sk] */
  const void* obias;    /* LF_BIAS & 2: additive output bias [B, Hq, Sq, D] */
  const void* q2;       /* LF_D2: second score product Q2 [B, Hq, Sq, D2] ... */
  const void* k2;       /* ... K2 [B, Hq / k2_group, Sk, D2] */
  int64_t q_sb, q_sh, q_ss;
  int64_t k_sb, k_sh, k_ss;   /* paged: k_sb = page stride, k_ss = token stride inside a page */
  int64_t v_sb, v_sh, v_ss;
  int64_t o_sb, o_sh, o_ss;
  int64_t bias_sb, bias_sh, bias_sq;   /* 0 = broadcast */
  int64_t ob_sb, ob_sh, ob_sq;
  int64_t q2_sb, q2_sh, q2_ss;
  int64_t k2_sb, k2_sh, k2_ss;
  int64_t k_span, v_span;     /* paged: elements from the pool's base pointer to the end of the pool */
  int32_t B, Hq, Hkv, Sq, Sk;
  int32_t window;             /* sliding-window width (LF_MASK == 2) */
  int32_t kt_stride, vt_stride;
  int32_t nsplit, rows, split_len;   /* decode */
  int32_t k2_group;
  float scale;                /* multiplies Q K^T */
  float softcap;              /* LF_SOFTCAP: cap of cap * tanh(s / cap) */
  float denom_add;            /* LF_DENOM: softmax denominator is sum + denom_add */
} LfAttnParamsHost;

/*
 * Parameter block of the backward kernels lf_attn_bwd_delta, lf_attn_bwd_dkdv and
 * lf_attn_bwd_dq (loopfuse_amd/csrc/kernels/lf_attn_bwd.hip, `struct LfAttnBwdParams`;
 * loopfuse_amd/lowering.py::AttnBwdParams is the ctypes mirror).  The three kernels take
 * the same block and run in that order on one stream.  The reference has no backward:
 * its backend traces inference graphs only (reference loopfuse/torch_backend/interface.py:600-621).
 */
typedef struct LfAttnBwdParamsHost {
  const void* q;        /* Q [B, Hq, Sq, D] */
  const void* k;        /* K [B, Hkv, Sk, D] */
  const void* v;
  const void* o;        /* the forward's output */
  const void* dout;     /* gradient of the output */
  void* dq;
  void* dk;             /* [B, Hkv, Sk, D]: summed over the query heads of a group */
  void* dv;
  const float* lse;     /* [B, Hq, Sq] row log-sum-exp of the scaled, masked scores in log2 units (part_ml of the forward) */
  float* delta;         /* [B, Hq, Sq] scratch, written by lf_attn_bwd_delta */
  int64_t q_sb, q_sh, q_ss;
  int64_t k_sb, k_sh, k_ss;
  int64_t v_sb, v_sh, v_ss;
  int64_t o_sb, o_sh, o_ss;
  int64_t do_sb, do_sh, do_ss;
  int64_t dq_sb, dq_sh, dq_ss;
  int64_t dk_sb, dk_sh, dk_ss;
  int64_t dv_sb, dv_sh, dv_ss;
  int32_t B, Hq, Hkv, Sq, Sk;
  int32_t window;       /* sliding-window width (LF_MASK == 2) */
  float scale;
  float softcap;        /* LF_SOFTCAP: cap of cap * tanh(s / cap) */
} LfAttnBwdParamsHost;

#ifdef __cplusplus
static_assert(sizeof(LfAttnBwdParamsHost) == 304, "LfAttnBwdParamsHost must match the device struct");
#else
_Static_assert(sizeof(LfAttnBwdParamsHost) == 304, "LfAttnBwdParamsHost must match the device struct");
#endif

#ifdef __cplusplus
static_assert(sizeof(LfAttnParamsHost) == 376, "LfAttnParamsHost must match the device struct");
}
#else
_Static_assert(sizeof(LfAttnParamsHost) == 376, "LfAttnParamsHost must match the device struct");
#endif

#endif /* LF_ATTN_PARAMS_H */
