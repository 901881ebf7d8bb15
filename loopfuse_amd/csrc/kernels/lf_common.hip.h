// lf_common.hip.h — shared device-side building blocks for the gfx950 attention
// kernels: element/vector types, the kernel parameter block, MFMA wrappers,
// cross-half-wave exchange, fast exp2/tanh and K/V row addressing (contiguous or
// gathered through a page table).
//
// Compile-time specialisation (passed as -D options by the host lowering):
//   LF_DTYPE      0 = bf16, 1 = fp16 storage (accumulation is always fp32)
//   LF_HEAD_DIM   64 or 128
//   LF_MASK       0 = none, 1 = causal (j <= i), 2 = causal sliding window
//                 (j <= i and i - j < window); top-left aligned as in the
//                 reference (loopfuse/torch_backend/ops.py:675-751)
//   LF_SOFTCAP    1: s <- cap * tanh(s * scale / cap) before the mask
//   LF_PAGED      bit 0: K rows, bit 1: V rows are gathered through a page table
//   LF_TABLE_I64  1: page tables hold int64 ids (else int32)
//   LF_PAGE_SIZE  tokens per page (power of two) when LF_PAGED
#ifndef LF_COMMON_HIP_H
#define LF_COMMON_HIP_H

#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif

#ifndef LF_DTYPE
#define LF_DTYPE 0
#endif
#ifndef LF_HEAD_DIM
#define LF_HEAD_DIM 128
#endif
#ifndef LF_MASK
#define LF_MASK 0
#endif
#ifndef LF_BIAS
#define LF_BIAS 0     /* bit 0: score bias tensor, bit 1: output bias tensor, bit 2: their rows are not
                         8-byte aligned (element loads); lf_attn_prefill only */
#endif
#ifndef LF_DENOM
#define LF_DENOM 0    /* 1: softmax denominator is (sum + denom_add) in units where the row maximum
                         contributes 1 (reference tests/test_attention.py:95-125); lf_attn_prefill only */
#endif
#ifndef LF_SOFTCAP
#define LF_SOFTCAP 0
#endif
#ifndef LF_PAGED
#define LF_PAGED 0
#endif
#ifndef LF_PAGE_SIZE
#define LF_PAGE_SIZE 16
#endif
#ifndef LF_PAGE_SIZE_V
#define LF_PAGE_SIZE_V LF_PAGE_SIZE   /* tokens per page of the V pool (K and V pools may differ) */
#endif
#ifndef LF_TABLE_I64
#define LF_TABLE_I64 0
#endif

#if LF_DTYPE == 0
typedef __bf16 lf_elem;
#else
typedef _Float16 lf_elem;
#endif

typedef lf_elem lf_elem8 __attribute__((ext_vector_type(8)));
typedef lf_elem lf_elem4 __attribute__((ext_vector_type(4)));
typedef lf_elem lf_elem2 __attribute__((ext_vector_type(2)));
typedef short lf_s16x4 __attribute__((ext_vector_type(4)));
typedef float lf_f32x2 __attribute__((ext_vector_type(2)));
typedef float lf_f32x4 __attribute__((ext_vector_type(4)));
typedef float lf_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int lf_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int lf_u32x2 __attribute__((ext_vector_type(2)));
typedef const int __attribute__((address_space(4))) lf_cint;   /* read-only table entries fetched with scalar loads */

#if LF_TABLE_I64
typedef long long lf_table_t;
#else
typedef int lf_table_t;
#endif

#define LF_NEG_INF (-__builtin_inff())
#define LF_LOG2E 1.4426950408889634f

// 1 / l for the final normalisation.  -DLF_SAFE=1: a query row that saw no key at all
// (l == 0: every score was -inf) comes out as zeros, which is what torch's fused attention
// ops return for it; the default is 0 * inf = NaN, what softmax of a row of -inf gives.
#ifndef LF_SAFE
#define LF_SAFE 0
#endif
// Score-bias values that mark a key as masked, for the searches that leave keys out which
// no query row can see (16-bit patterns; the second form takes two packed values).  -inf
// always.  With LF_SAFE also the finite values masks are commonly filled with, the most
// negative finite number of the storage type and its binade (<= -1.7e38 for bf16,
// <= -57344 for fp16): next to any visible key their probabilities underflow to exactly 0,
// so leaving them out changes nothing for a row that sees a key; a row that sees none
// gives zeros under LF_SAFE either way.  NaN never counts.
__device__ __forceinline__ bool lf_bias_masked(unsigned bits) {
  constexpr unsigned kNegInf = LF_DTYPE == 0 ? 0xff80u : 0xfc00u;
#if LF_SAFE
  constexpr unsigned kFloor = LF_DTYPE == 0 ? 0xff00u : 0xfb00u;
  return bits >= kFloor && bits <= kNegInf;
#else
  return bits == kNegInf;
#endif
}
__device__ __forceinline__ bool lf_bias_masked2(unsigned raw) {
  return lf_bias_masked(raw & 0xffffu) && lf_bias_masked(raw >> 16);
}

// Value a score-bias element adds to a score.  With LF_SAFE the values that count as masked
// (see above) add -inf, so a key gets probability exactly 0 whether its tile / span was walked
// or left out: a row that sees no key then gives zeros in every case.
__device__ __forceinline__ float lf_bias_value(lf_elem b) {
#if LF_SAFE
  return lf_bias_masked(__builtin_bit_cast(unsigned short, b)) ? LF_NEG_INF : (float)b;
#else
  return (float)b;
#endif
}

__device__ __forceinline__ float lf_inv_sum(float l) {
#if LF_SAFE
  return l > 0.0f ? 1.0f / l : 0.0f;
#else
  return 1.0f / l;
#endif
}

// Kernel parameter block.  Mirrors loopfuse_amd/lowering.py::AttnParams field
// for field (pointers, then 64-bit element strides, then 32-bit scalars).
struct LfAttnParams {
  const lf_elem* q;
  const lf_elem* k;          // contiguous K, or the K page pool when LF_PAGED
  const lf_elem* v;
  lf_elem* o;
  const void* k_table;       // [B, pages_per_seq] page ids (lf_table_t) when paged
  const void* v_table;
  float* part_acc;           // split-K scratch: [units, nsplit, rows, D]; prefill_swp with LF_BIAS: the bias tile classes (int32)
  float* part_ml;            // split-K scratch: [units, nsplit, rows, 2] (max, sum); lf_attn_prefill_swp: optional
                             // output [B, Hq, Sq], the rows' log-sum-exp in log2 units (null: not written)
  unsigned char* visits;     // optional [B*Hq*nqt, nkt] visited-tile record
  const lf_elem* bias;       // LF_BIAS & 1: additive score bias [B, Hq, Sq, Sk] (key stride 1),
                             // added after scale / softcap and before the mask
  const lf_elem* obias;      // LF_BIAS & 2: additive output bias [B, Hq, Sq, D] (d stride 1)
  const lf_elem* q2;         // LF_D2: second score product, scores = Q K^T + Q2 K2^T (the two-part
  const lf_elem* k2;         // scores of reference tests/test_attention.py:126-151); dense, depth LF_D2
  long long q_sb, q_sh, q_ss;  // element strides of Q [B, Hq, Sq, D] (d stride 1)
  long long k_sb, k_sh, k_ss;  // K [B, Hkv, Sk, D]; paged: k_sb = page stride,
                               // k_ss = stride between tokens inside a page
  long long v_sb, v_sh, v_ss;
  long long o_sb, o_sh, o_ss;
  long long bias_sb, bias_sh, bias_sq;   // element strides of bias (0 = broadcast)
  long long ob_sb, ob_sh, ob_sq;         // element strides of obias (0 = broadcast)
  long long q2_sb, q2_sh, q2_ss;         // Q2 [B, Hq, Sq, LF_D2] (d stride 1)
  long long k2_sb, k2_sh, k2_ss;         // K2 [B, Hq / k2_group, Sk, LF_D2] (d stride 1)
  long long k_span, v_span;              // paged: elements from the pool's base to its end (the range the
                                         // direct-to-LDS loads are checked against)
  int B, Hq, Hkv, Sq, Sk;
  int window;                // sliding-window width (LF_MASK == 2)
  int kt_stride, vt_stride;  // row strides (elements) of k_table / v_table
  int nsplit;                // decode: number of KV splits across workgroups
  int rows;                  // decode: query rows per (batch, kv head) unit
  int split_len;             // decode: tokens per split (multiple of 16)
  int k2_group;              // LF_D2: query heads per K2 head
  float scale;               // multiplies QK^T (D^-0.5 in the reference graphs)
  float softcap;             // cap of cap*tanh(s/cap) (LF_SOFTCAP)
  float denom_add;           // LF_DENOM: probabilities are e^(x - max) / (sum e^(x - max) + denom_add)
};

__device__ __forceinline__ lf_f32x16 lf_mfma32(lf_elem8 a, lf_elem8 b, lf_f32x16 c) {
#if LF_DTYPE == 0
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#endif
}

__device__ __forceinline__ lf_f32x4 lf_mfma16(lf_elem8 a, lf_elem8 b, lf_f32x4 c) {
#if LF_DTYPE == 0
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
#endif
}

// 16x16x16: A lane (row = lane % 16, group = lane / 16) holds k = 4*group .. +3
__device__ __forceinline__ lf_f32x4 lf_mfma16k16(lf_elem4 a, lf_elem4 b, lf_f32x4 c) {
#if LF_DTYPE == 0
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(lf_s16x4, a), __builtin_bit_cast(lf_s16x4, b), c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
#endif
}

// Value held by the lane 32 positions away (lane l <-> lane l ^ 32): one
// v_permlane32_swap (VALU) instead of a round trip through the LDS crossbar.
__device__ __forceinline__ float lf_swap32(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  // swaps the upper half of the first operand with the lower half of the second:
  // with both operands = x, result[0] holds x of lane^32 in lanes 32..63 and
  // result[1] holds it in lanes 0..31
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned other = (__lane_id() < 32) ? r[1] : r[0];
  return __builtin_bit_cast(float, other);
}

// max(x of this lane, x of lane ^ 32) in every lane.  After v_permlane32_swap of two copies of x one register
// holds the lower half's values in both halves and the other the upper half's: their maximum is the answer
// without a select.  Inline asm: written with the builtin, the compiler keeps the swap and drops the maximum.
__device__ __forceinline__ float lf_max_halves(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}

__device__ __forceinline__ float lf_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// tanh(x) = 1 - 2 / (2^(2 x log2 e) + 1); exact limits at +-inf.
__device__ __forceinline__ float lf_tanh(float x) {
  float e = lf_exp2(x * (2.0f * LF_LOG2E));
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

__device__ __forceinline__ lf_elem lf_from_float(float x) { return (lf_elem)x; }
__device__ __forceinline__ float lf_to_float(lf_elem x) { return (float)x; }

// Pointer to element 0 of row `tok` of K (which = 0) or V (which = 1) for batch
// b and kv head h.  With LF_PAGED the row lives in page table[b][tok / P] of the
// pool, at token slot tok % P (reference semantics: out[*s,*t] =
// buffer[block_table[*s],*t], loopfuse/torch_backend/__init__.py:46-56).
__device__ __forceinline__ const lf_elem* lf_kv_row(const LfAttnParams& p, int which, int b, int h,
                                                   int tok) {
  const lf_elem* base = which ? p.v : p.k;
  const long long sb = which ? p.v_sb : p.k_sb;
  const long long sh = which ? p.v_sh : p.k_sh;
  const long long ss = which ? p.v_ss : p.k_ss;
  const bool paged = which ? ((LF_PAGED & 2) != 0) : ((LF_PAGED & 1) != 0);
  if (paged) {
    const lf_table_t* table = reinterpret_cast<const lf_table_t*>(which ? p.v_table : p.k_table);
    const int psz = which ? LF_PAGE_SIZE_V : LF_PAGE_SIZE;
    const long long page = table[(long long)b * (which ? p.vt_stride : p.kt_stride) + (tok / psz)];
    return base + page * sb + (long long)(tok % psz) * ss + (long long)h * sh;
  }
  return base + (long long)b * sb + (long long)h * sh + (long long)tok * ss;
}

#endif  // LF_COMMON_HIP_H
