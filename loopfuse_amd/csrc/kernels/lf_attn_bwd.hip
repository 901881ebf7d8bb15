// lf_attn_bwd.hip — backward of the fused attention forward (dense K/V, mask none / causal /
// sliding window, scale, optional softcap; no bias) for gfx950.  The reference has no backward
// (its README lists it as future work); the formulas are the standard ones for
// O = softmax(scale * Q K^T + mask) V with the row log-sum-exp L kept by the forward:
//   P = exp(scale * Q K^T - L),  dV = P^T dO,  dP = dO V^T,  delta = rowsum(dO * O),
//   dS = scale * P * (dP - delta),  dQ = dS K,  dK = dS^T Q.
// With a softcap (LF_SOFTCAP) the scores are T = cap * tanh(scale * Q K^T / cap), P = exp(T - L), and
// dS picks up the derivative of the cap: dS = scale * (1 - tanh^2) * P * (dP - delta).
// Three kernels, no atomics, every result written once (deterministic):
//   lf_attn_bwd_delta : delta[b, h, q]
//   lf_attn_bwd_dkdv  : a workgroup owns 128 keys of one (batch, kv head) -- 4 waves x 32 keys,
//                       K^T and V^T of its keys in registers as MFMA B operands -- and walks the
//                       q tiles (64 rows) of the query heads of the group that can see them
//   lf_attn_bwd_dq    : a workgroup owns 128 query rows of one (batch, head), Q^T and dO^T in
//                       registers, and walks the kv tiles (64 keys) as the forward does
// The tiles that are walked go through LDS in the two layouts of lf_prefill_blocks.hip.h: the
// K layout (ds_read_b128, rows of the tile = MFMA rows) and the V layout (transposed reads,
// rows of the tile = MFMA k).  As in the forward, the accumulator of the first product is, as
// held, the B operand of the second, so P and dS never leave registers.
// L and the exponent are in log2 units (the forward writes L2 = offset + log2(sum)).

struct LfAttnBwdParams {
  const lf_elem* q;       // [B, Hq, Sq, D]
  const lf_elem* k;       // [B, Hkv, Sk, D]
  const lf_elem* v;
  const lf_elem* o;       // forward output
  const lf_elem* dout;    // gradient of the output
  lf_elem* dq;
  lf_elem* dk;
  lf_elem* dv;
  const float* lse;       // [B, Hq, Sq] row log-sum-exp of the scaled, masked scores, log2 units
  float* delta;           // [B, Hq, Sq] scratch: rowsum(dO * O)
  long long q_sb, q_sh, q_ss;      // element strides (d stride 1)
  long long k_sb, k_sh, k_ss;
  long long v_sb, v_sh, v_ss;
  long long o_sb, o_sh, o_ss;
  long long do_sb, do_sh, do_ss;
  long long dq_sb, dq_sh, dq_ss;
  long long dk_sb, dk_sh, dk_ss;
  long long dv_sb, dv_sh, dv_ss;
  int B, Hq, Hkv, Sq, Sk;
  int window;
  float scale;
  float softcap;          // LF_SOFTCAP: cap of cap * tanh(s / cap)
};

#define LF_BW_NT 256
#ifndef LF_BW_GROUP
#define LF_BW_GROUP 4      /* (batch, kv head) pairs of one XCD whose workgroups are dispatched together */
#endif
// Is the score with (query - key) = t kept?  Callers fold the bound of the key sequence into t.
__device__ __forceinline__ bool lf_bw_keep(int t, int window) {
#if LF_MASK == 0
  (void)window;
  return t > -(1 << 29);
#elif LF_MASK == 1
  (void)window;
  return t >= 0;
#else
  return (unsigned)t < (unsigned)window;
#endif
}
#ifndef LF_BW_DQ_NT
#define LF_BW_DQ_NT 512     /* threads of lf_attn_bwd_dq: 8 waves x 32 query rows, two waves per SIMD */
#endif

// delta[row] = sum_d dO[row][d] * O[row][d]; 16 lanes per row, 8 elements per lane
extern "C" __global__ void __launch_bounds__(LF_BW_NT) lf_attn_bwd_delta(const LfAttnBwdParams p) {
  const long long row = (long long)blockIdx.x * (LF_BW_NT / 16) + threadIdx.x / 16;
  const int piece = threadIdx.x % 16;
  const long long nrows = (long long)p.B * p.Hq * p.Sq;
  float s = 0.0f;
  if (row < nrows && piece < LF_CPR) {
    const int qi = (int)(row % p.Sq);
    const int h = (int)((row / p.Sq) % p.Hq);
    const int b = (int)(row / ((long long)p.Sq * p.Hq));
    const lf_elem8 ov = *reinterpret_cast<const lf_elem8*>(p.o + b * p.o_sb + h * p.o_sh + qi * p.o_ss + 8 * piece);
    const lf_elem8 gv = *reinterpret_cast<const lf_elem8*>(p.dout + b * p.do_sb + h * p.do_sh + qi * p.do_ss + 8 * piece);
#pragma unroll
    for (int e = 0; e < 8; ++e) s += (float)ov[e] * (float)gv[e];
  }
  s += __shfl_xor(s, 1, 64);
  s += __shfl_xor(s, 2, 64);
  s += __shfl_xor(s, 4, 64);
  s += __shfl_xor(s, 8, 64);
  if (row < nrows && piece == 0) p.delta[row] = s;
}

// A 64-row tile of a [rows, D] matrix goes global -> LDS directly (buffer_load ... lds, the
// forward's staging): per pass the workgroup's NT threads move NT / LF_CPR whole rows, a wave
// 64 lanes x 16 B that land contiguously; the XOR swizzle of the K layout (`tr` false:
// ds_read_b128, tile rows = MFMA rows) or of the V layout (`tr` true: transposed reads, tile
// rows = MFMA k) is applied on the global side.  `rs` covers rows 0 .. nrows-1 of the matrix
// (row stride `rowb` bytes): rows past the end get an offset beyond it and arrive as zeros.
// Not tracked by the compiler's wait counters: callers wait with s_waitcnt vmcnt(0).
template <int NT>
__device__ __forceinline__ unsigned lf_bw_dma_lane_off(unsigned rowb, bool tr, int tid) {
  // byte offset of this lane's 16 bytes in the first pass of a tile that starts at row 0; the
  // swizzles repeat every 16 rows and a pass is a multiple of 16 rows, so every pass adds rows only
  const int srow = tid / LF_CPR, sch = tid % LF_CPR;
  return (unsigned)srow * rowb + 16u * (unsigned)(tr ? lf_v_phys(srow, sch) : lf_k_phys(srow, sch));
}
template <int NT>
__device__ __forceinline__ void lf_bw_dma_piece(const lf_u32x4& rs, unsigned rowb, int row0, lf_elem* tile,
                                                unsigned lane_off, int ps, int wave) {
  constexpr int kRowsPerPass = NT / LF_CPR, kRowsPerWave = 64 / LF_CPR;
  static_assert(kRowsPerPass % 16 == 0, "a pass must keep the swizzle phase");
  const unsigned off = (unsigned)(row0 + kRowsPerPass * ps) * rowb + lane_off;
  lf_dma_to_lds(rs, off, &tile[(kRowsPerPass * ps + kRowsPerWave * wave) * LF_D]);
}
// wait for this wave's direct loads and LDS writes, then meet the other waves.  The wait is the
// builtin, not inline asm, so that the compiler's wait-counter pass sees that nothing is
// outstanding afterwards: otherwise it waits again inside the step -- for the operands loaded
// before the loop and before overwriting a register a tracked load wrote -- with vmcnt values
// that also drain the direct loads of the next stage just issued (0x0070: vmcnt(0) lgkmcnt(0))
#define LF_BW_BARRIER()                      \
  do {                                       \
    asm volatile("" ::: "memory");           \
    __builtin_amdgcn_s_waitcnt(0x0070);      \
    __builtin_amdgcn_s_barrier();            \
    asm volatile("" ::: "memory");           \
  } while (0)

// Fragment read-ahead of the two product loops (LDS reads in flight ahead of the MFMA that
// consumes them; the order of reads and MFMAs is pinned with scheduling barriers, left to
// itself the compiler issues read, wait, MFMA one after the other)
#define LF_BW_PF1 3      /* first products: pairs of K-layout fragments */
#define LF_BW_PF2 4      /* second products: V-layout fragments */
#define LF_BW_DQ_PF1 2   /* lf_attn_bwd_dq, first products: 3 do not fit its 256 registers */

// MFMAs of lf_attn_bwd_dkdv with the register file of every operand spelled out.  At one wave per
// SIMD the kernel has 512 registers per lane, and the compiler then gives every MFMA an AGPR
// destination while keeping what it computes with in VGPRs: left to it, the loop carries hundreds
// of v_accvgpr moves per step.  Here dK^T / dV^T (written in the loop, read after it) and the
// loop-invariant K^T / V^T operands live in AGPRs, S^T / dP^T (read by the VALU right away) in VGPRs.
// What the compiler would otherwise see to: an MFMA result may be read 12 wait states after the MFMA
// was issued at the earliest (LF_BW_MFMA_DRAIN), and a VGPR written by the VALU may be an MFMA
// operand 2 wait states later (LF_BW_VALU_SETTLE); back-to-back MFMAs on one accumulator need nothing.
// What it cannot see to at all: a register copy or a spill of its own placed right behind one of these
// MFMAs would read the accumulator too early.  The live ranges are laid out so that it has no reason
// for either, and tests/test_kernel_codegen.py checks the generated code for it.
#if LF_DTYPE == 0
#define LF_BW_MFMA "v_mfma_f32_32x32x16_bf16"
#else
#define LF_BW_MFMA "v_mfma_f32_32x32x16_f16"
#endif
#define LF_BW_MFMA_DRAIN "s_nop 9\n\ts_nop 9"
#define LF_BW_MFMA_DRAIN_LAST "s_nop 15\n\ts_nop 15\n\ts_nop 15"     /* behind the last MFMAs issued: one may still wait for the pipe */
#define LF_BW_VALU_SETTLE "s_nop 1"
// c (VGPRs) = a (VGPRs) x b (AGPRs)
__device__ __forceinline__ void lf_bw_mfma_first(lf_f32x16& c, const lf_u32x4& a, const lf_u32x4& b) {
  asm volatile(LF_BW_MFMA " %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
}
// c (VGPRs) += a (VGPRs) x b (AGPRs)
__device__ __forceinline__ void lf_bw_mfma_vva(lf_f32x16& c, const lf_u32x4& a, const lf_u32x4& b) {
  asm volatile(LF_BW_MFMA " %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
}
// c (AGPRs) += a (VGPRs) x b (VGPRs)
__device__ __forceinline__ void lf_bw_mfma_avv(lf_f32x16& c, const lf_u32x4& a, const lf_u32x4& b) {
  asm volatile(LF_BW_MFMA " %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// lf_attn_bwd_dq in its 8-wave form runs two waves per SIMD on 256 registers: the compiler then uses
// no AGPRs and its own MFMAs are as good; the 4-wave form has 512 and gets the explicit ones
#if LF_BW_DQ_NT == 256
#define LF_BW_DQ_ASM 1
#else
#define LF_BW_DQ_ASM 0
#endif
__device__ __forceinline__ void lf_bw_dq_mfma_s(lf_f32x16& c, const lf_u32x4& a, const lf_u32x4& b, bool first) {
#if LF_BW_DQ_ASM
  if (first) lf_bw_mfma_first(c, a, b); else lf_bw_mfma_vva(c, a, b);
#else
  if (first) {
#pragma unroll
    for (int i = 0; i < 16; ++i) c[i] = 0.0f;
  }
  c = lf_mfma32(__builtin_bit_cast(lf_elem8, a), __builtin_bit_cast(lf_elem8, b), c);
#endif
}
__device__ __forceinline__ void lf_bw_dq_mfma_acc(lf_f32x16& c, const lf_u32x4& a, const lf_u32x4& b) {
#if LF_BW_DQ_ASM
  lf_bw_mfma_avv(c, a, b);
#else
  c = lf_mfma32(__builtin_bit_cast(lf_elem8, a), __builtin_bit_cast(lf_elem8, b), c);
#endif
}

// accumulators X^T[d][n] (lane n = lane % 32; element i of block db is d = 32*db + 8*(i/4) + 4*g + i%4)
// -> rows n of a [rows, D] matrix, 16 bytes per store (the exchange of the forward's epilogue)
__device__ __forceinline__ void lf_bw_store_rows(const lf_f32x16* acc, lf_elem* row_ptr, bool valid, int g) {
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db) {
    unsigned ch[4][2];
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      lf_elem4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = lf_from_float(acc[db][4 * i4 + e]);
      const lf_u32x2 wu = __builtin_bit_cast(lf_u32x2, w);
      ch[i4][0] = wu[0];
      ch[i4][1] = wu[1];
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      auto r0 = __builtin_amdgcn_permlane32_swap(ch[2 * j][0], ch[2 * j + 1][0], false, false);
      auto r1 = __builtin_amdgcn_permlane32_swap(ch[2 * j][1], ch[2 * j + 1][1], false, false);
      const lf_u32x4 out = {r0[0], r1[0], r0[1], r1[1]};
      if (valid) *reinterpret_cast<lf_u32x4*>(row_ptr + 32 * db + 16 * j + 8 * g) = out;
    }
  }
}

extern "C" __global__ void __launch_bounds__(LF_BW_NT, 1) lf_attn_bwd_dkdv(const LfAttnBwdParams p) {
  // two stages of: Q tile in both layouts, dO tile in both layouts, L and delta of the 64 rows
  __shared__ __attribute__((aligned(16))) lf_elem tiles[2][4][64 * LF_D];
  __shared__ __attribute__((aligned(16))) float lse_st[2][64];
  __shared__ __attribute__((aligned(16))) float delta_st[2][64];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int g = lane >> 5;

  const int nkt = (p.Sk + 127) / 128;
  // Workgroup ids with equal id % 8 run on one XCD.  All key blocks of a (batch, kv head) go to one
  // XCD, so the Q / dO tiles they all walk are fetched into one L2, once; within an XCD the ids come
  // in groups of LF_BW_GROUP (batch, kv head) pairs and, inside a group, by key block, the ones with
  // the most steps under a causal mask first.  The grid is padded to whole groups.
  const int slot = blockIdx.x / 8;
  const int in_grp = slot % (LF_BW_GROUP * nkt);
  const int kt = in_grp / LF_BW_GROUP;
  const int bhkv = (slot / (LF_BW_GROUP * nkt) * LF_BW_GROUP + in_grp % LF_BW_GROUP) * 8 + (int)(blockIdx.x % 8);
  if (bhkv >= p.B * p.Hkv) return;
  const int hkv = bhkv % p.Hkv;
  const int b = bhkv / p.Hkv;
  const int group = p.Hq / p.Hkv;
  const int key0 = 128 * kt + 32 * wave;           // first key of this wave
  const int my_key = key0 + l32;
  const int nqt = (p.Sq + 63) / 64;

  // K^T and V^T of this lane's key as B operands (d = 16*ks + 8*g .. +7), parked in AGPRs
  lf_u32x4 kf[LF_NKS], vf[LF_NKS];
  {
    const int kr = min(my_key, p.Sk - 1);
    const lf_elem* krow = p.k + (long long)b * p.k_sb + (long long)hkv * p.k_sh + (long long)kr * p.k_ss;
    const lf_elem* vrow = p.v + (long long)b * p.v_sb + (long long)hkv * p.v_sh + (long long)kr * p.v_ss;
#pragma unroll
    for (int ks = 0; ks < LF_NKS; ++ks) {
      kf[ks] = *reinterpret_cast<const lf_u32x4*>(krow + 16 * ks + 8 * g);
      vf[ks] = *reinterpret_cast<const lf_u32x4*>(vrow + 16 * ks + 8 * g);
    }
#pragma unroll
    for (int ks = 0; ks < LF_NKS; ++ks) asm volatile("" : "+a"(kf[ks]), "+a"(vf[ks]));
  }
#if LF_SOFTCAP
  const float sc_exp = p.scale / p.softcap * (2.0f * LF_LOG2E);   // 2^(s * sc_exp) = e^(2x)
  const float cexp = p.softcap * LF_LOG2E;                        // exponent of P: tanh x * cexp - L
#else
  const float cexp = p.scale * LF_LOG2E;
#endif

  lf_f32x16 dk[LF_NDB], dv[LF_NDB];
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db) {
#pragma unroll
    for (int i = 0; i < 16; ++i) dk[db][i] = dv[db][i] = 0.0f;
    asm volatile("" : "+a"(dk[db]), "+a"(dv[db]));
  }

  // q tiles (64 rows) that hold a query seeing one of the workgroup's 128 keys
  int qt_begin = 0, qt_end = nqt;
#if LF_MASK >= 1
  qt_begin = (128 * kt) / 64;                                   // q >= key
#endif
#if LF_MASK == 2
  qt_end = min(nqt, (min(128 * kt + 127, p.Sk - 1) + p.window - 1) / 64 + 1);   // q - key < window
#endif

  // the steps of this workgroup: query heads of the group x q tiles, one flat sequence; the
  // direct loads of step it + 1 fill the other stage while step it is computed, one load after
  // every pair of MFMAs of the first products (a wave owes LF_CPR loads per step, and that many
  // pairs there are: the loads go through the CU's one texture path at 64 bytes per cycle, issued
  // in one go they hold up the wave for as long as a quarter of its MFMAs take)
  const int ntq = max(qt_end - qt_begin, 0);
  const int nsteps = group * ntq;
  const unsigned q_bytes = (unsigned)(((long long)(p.Sq - 1) * p.q_ss + LF_D) * 2);
  const unsigned g_bytes = (unsigned)(((long long)(p.Sq - 1) * p.do_ss + LF_D) * 2);
  const int wave_u = wave;
  constexpr int kPasses = 64 * LF_CPR / LF_BW_NT;      // loads of a wave per tile
  static_assert(4 * kPasses == 2 * LF_NKS, "one direct load per pair of MFMAs of the first products");
  float r_lse = 0.0f, r_delta = 0.0f;
  lf_u32x4 q_rs, g_rs;        // rows of Q and dO of the step being loaded (zero bytes: nothing to load)
  int q0_next = 0;
  auto aim = [&](int it, bool real) {
    const int h = hkv * group + it / ntq;
    q0_next = 64 * (qt_begin + it % ntq);
    q_rs = lf_make_buffer(p.q + (long long)b * p.q_sb + (long long)h * p.q_sh, real ? q_bytes : 0u);
    g_rs = lf_make_buffer(p.dout + (long long)b * p.do_sb + (long long)h * p.do_sh, real ? g_bytes : 0u);
    if (tid < 64) {            // into registers now, into the stage just before the barrier that opens it
      const long long r = ((long long)b * p.Hq + h) * p.Sq + q0_next + tid;
      const bool in = real && q0_next + tid < p.Sq;
      r_lse = in ? p.lse[r] : __builtin_inff();                      // rows past Sq: P = 0
      r_delta = in ? p.delta[r] : 0.0f;
    }
  };
  const unsigned lane_off[4] = {lf_bw_dma_lane_off<LF_BW_NT>((unsigned)p.q_ss * 2u, false, tid),
                                lf_bw_dma_lane_off<LF_BW_NT>((unsigned)p.q_ss * 2u, true, tid),
                                lf_bw_dma_lane_off<LF_BW_NT>((unsigned)p.do_ss * 2u, false, tid),
                                lf_bw_dma_lane_off<LF_BW_NT>((unsigned)p.do_ss * 2u, true, tid)};
  auto issue_piece = [&](int st, int j) {      // load j of LF_CPR: tile j / kPasses (Q, Q, dO, dO), pass j % kPasses
    const int t = j / kPasses;
    lf_bw_dma_piece<LF_BW_NT>(t < 2 ? q_rs : g_rs, (unsigned)(t < 2 ? p.q_ss : p.do_ss) * 2u, q0_next, tiles[st][t],
                              lane_off[t], j % kPasses, wave_u);
  };
  auto publish = [&](int st) {
    if (tid < 64) {
      lse_st[st][tid] = r_lse;
      delta_st[st][tid] = r_delta;
    }
  };
  // One step of a wave: S^T and dP^T of 32 keys x 64 queries in two blocks of 32 queries, P and dS,
  // then dV^T += dO^T P and dK^T += Q^T dS.  With one wave per SIMD nothing else fills the matrix
  // pipe while the wave computes P and dS, so the step is written as four phases of 16 MFMAs with
  // that arithmetic placed between them: first products of block 0 | first products of block 1 with
  // P, dS of block 0 | second products over block 0's queries with P, dS of block 1 | second
  // products over block 1's queries.  dS is kept without the factor `scale`, which multiplies dK once
  // at the end.
  auto step = [&](bool masked, int st, int q0) {
    // query minus key of element (qb, i4, e) is rel + 32*qb + 8*i4 + e; a key past Sk fails every test
    const int rel = my_key < p.Sk ? q0 + 4 * g - my_key : -(1 << 30);
    const lf_elem* q_rm = tiles[st][0];
    const lf_elem* q_tr = tiles[st][1];
    const lf_elem* g_rm = tiles[st][2];
    const lf_elem* g_tr = tiles[st][3];
    const float* lse_s = lse_st[st];
    const float* delta_s = delta_st[st];
    constexpr int kNF = LF_NKK * LF_NDB;
    lf_u32x4 pf[LF_NKK], dsf[LF_NKK];
    lf_f32x16 s[2], dp[2];
    // P and dS of the four queries (qb, i4): elements 4*i4 .. +3 of the accumulators, query
    // q0 + 32*qb + 8*i4 + 4*g + e, key my_key
    auto soft4 = [&](int qb, int i4) {
      const int ql = 32 * qb + 8 * i4 + 4 * g;
      const lf_f32x4 l4 = *reinterpret_cast<const lf_f32x4*>(&lse_s[ql]);
      const lf_f32x4 d4 = *reinterpret_cast<const lf_f32x4*>(&delta_s[ql]);
      lf_elem4 pw, dw;
      float pv[4];
#if LF_SOFTCAP
      float dcap[4];           // 1 - tanh^2
#endif
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * i4 + e;
#if LF_SOFTCAP
        const float r = __builtin_amdgcn_rcpf(1.0f + lf_exp2(s[qb][i] * sc_exp));     // 1 / (e^(2x) + 1), x = s * scale / cap
        const float th = 1.0f - 2.0f * r;                                               // tanh x
        pv[e] = lf_exp2(th * cexp - l4[e]);
        dcap[e] = 4.0f * r * (1.0f - r);
#else
        pv[e] = lf_exp2(s[qb][i] * cexp - l4[e]);
#endif
      }
      if (masked) {             // wave-uniform: most steps of a workgroup lie below the diagonal
#pragma unroll
        for (int e = 0; e < 4; ++e) pv[e] = lf_bw_keep(rel + 32 * qb + 8 * i4 + e, p.window) ? pv[e] : 0.0f;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * i4 + e;
        pw[e] = lf_from_float(pv[e]);
#if LF_SOFTCAP
        dw[e] = lf_from_float(pv[e] * (dp[qb][i] - d4[e]) * dcap[e]);
#else
        dw[e] = lf_from_float(pv[e] * (dp[qb][i] - d4[e]));
#endif
      }
      const lf_u32x2 pu = __builtin_bit_cast(lf_u32x2, pw), du = __builtin_bit_cast(lf_u32x2, dw);
      pf[2 * qb + i4 / 2][2 * (i4 % 2)] = pu[0];
      pf[2 * qb + i4 / 2][2 * (i4 % 2) + 1] = pu[1];
      dsf[2 * qb + i4 / 2][2 * (i4 % 2)] = du[0];
      dsf[2 * qb + i4 / 2][2 * (i4 % 2) + 1] = du[1];
    };
    // phases 1 and 2
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      lf_u32x4 qa[LF_NKS], ga[LF_NKS];
#pragma unroll
      for (int ks = 0; ks < LF_BW_PF1; ++ks) {
        qa[ks] = lf_read_k_frag(q_rm, l32, g, ks * LF_NKB + qb);
        ga[ks] = lf_read_k_frag(g_rm, l32, g, ks * LF_NKB + qb);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < LF_NKS; ++ks) {
        if (ks + LF_BW_PF1 < LF_NKS) {
          qa[ks + LF_BW_PF1] = lf_read_k_frag(q_rm, l32, g, (ks + LF_BW_PF1) * LF_NKB + qb);
          ga[ks + LF_BW_PF1] = lf_read_k_frag(g_rm, l32, g, (ks + LF_BW_PF1) * LF_NKB + qb);
        }
        if (ks == 0) {
          lf_bw_mfma_first(s[qb], qa[ks], kf[ks]);
          lf_bw_mfma_first(dp[qb], ga[ks], vf[ks]);
        } else {
          lf_bw_mfma_vva(s[qb], qa[ks], kf[ks]);
          lf_bw_mfma_vva(dp[qb], ga[ks], vf[ks]);
        }
        issue_piece(st ^ 1, LF_NKS * qb + ks);
        if (qb == 1 && ks * 4 % LF_NKS == 0) soft4(0, ks * 4 / LF_NKS);      // 4 groups over the LF_NKS pairs
        __builtin_amdgcn_sched_barrier(0);
      }
      asm volatile(LF_BW_MFMA_DRAIN : "+v"(s[qb]), "+v"(dp[qb]));
    }
    // phases 3 and 4
    {
      lf_u32x4 gt[kNF], qt2[kNF];
#pragma unroll
      for (int f = 0; f < LF_BW_PF2; ++f) {
        gt[f] = __builtin_bit_cast(lf_u32x4, lf_read_v_frag_tr(g_tr, lane, g, f));
        qt2[f] = __builtin_bit_cast(lf_u32x4, lf_read_v_frag_tr(q_tr, lane, g, f));
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int f = 0; f < kNF; ++f) {
        if (f % (kNF / 2) == 0) {
#pragma unroll
          for (int kk = 0; kk < LF_NKK / 2; ++kk)
            asm volatile(LF_BW_VALU_SETTLE : "+v"(pf[f / (kNF / 2) * (LF_NKK / 2) + kk]), "+v"(dsf[f / (kNF / 2) * (LF_NKK / 2) + kk]));
        }
        if (f + LF_BW_PF2 < kNF) {
          gt[f + LF_BW_PF2] = __builtin_bit_cast(lf_u32x4, lf_read_v_frag_tr(g_tr, lane, g, f + LF_BW_PF2));
          qt2[f + LF_BW_PF2] = __builtin_bit_cast(lf_u32x4, lf_read_v_frag_tr(q_tr, lane, g, f + LF_BW_PF2));
        }
        lf_bw_mfma_avv(dv[f % LF_NDB], gt[f], pf[f / LF_NDB]);
        lf_bw_mfma_avv(dk[f % LF_NDB], qt2[f], dsf[f / LF_NDB]);
        if (f < kNF / 2 && f * 8 % kNF == 0) soft4(1, f * 8 / kNF);              // 4 groups over the first kNF / 2 pairs
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  if (nsteps > 0) {
    aim(0, true);
#pragma unroll
    for (int j = 0; j < LF_CPR; ++j) issue_piece(0, j);
    publish(0);
  }
  LF_BW_BARRIER();
  for (int it = 0; it < nsteps; ++it) {
    const int st = it & 1;
    const int q0 = 64 * (qt_begin + it % ntq);
    // the other stage was last read in step it - 1, which every wave left at the barrier below;
    // after the last step the loads still go out, against an empty range: they fetch nothing
    aim(min(it + 1, nsteps - 1), it + 1 < nsteps);

    bool need = key0 < p.Sk;
#if LF_MASK >= 1
    need = need && (q0 + 63 >= key0);
#endif
#if LF_MASK == 2
    need = need && (q0 - min(key0 + 31, p.Sk - 1) < p.window);
#endif
    if (need) {                 // wave-uniform
      // are all 32 x 64 scores of this wave kept?  Then the step runs without the mask arithmetic
      bool full = key0 + 31 < p.Sk;
#if LF_MASK >= 1
      full = full && (key0 + 31 <= q0);
#endif
#if LF_MASK == 2
      full = full && (q0 + 63 - key0 < p.window);
#endif
      step(!full, st, q0);
    } else {
#pragma unroll
      for (int j = 0; j < LF_CPR; ++j) issue_piece(st ^ 1, j);
    }
    if (it + 1 < nsteps) publish(st ^ 1);
    LF_BW_BARRIER();            // the next stage has landed; every wave is done with this one
  }
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db) asm volatile(LF_BW_MFMA_DRAIN_LAST : "+a"(dk[db]), "+a"(dv[db]));
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) dk[db][i] *= p.scale;

  const bool valid = my_key < p.Sk;
  const int kr = min(my_key, p.Sk - 1);
  lf_bw_store_rows(dk, p.dk + (long long)b * p.dk_sb + (long long)hkv * p.dk_sh + (long long)kr * p.dk_ss, valid, g);
  lf_bw_store_rows(dv, p.dv + (long long)b * p.dv_sb + (long long)hkv * p.dv_sh + (long long)kr * p.dv_ss, valid, g);
}

extern "C" __global__ void __launch_bounds__(LF_BW_DQ_NT, LF_BW_DQ_NT / 256) lf_attn_bwd_dq(const LfAttnBwdParams p) {
  // two stages of: K tile in both layouts, V tile in the K layout
  __shared__ __attribute__((aligned(16))) lf_elem tiles[2][3][64 * LF_D];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int g = lane >> 5;

  constexpr int kBM = LF_BW_DQ_NT / 2;                    // query rows of a workgroup
  const int nqt = (p.Sq + kBM - 1) / kBM;
  // As in lf_attn_bwd_dkdv: the q tiles of all query heads of a (batch, kv head) run on one XCD
  // and share its K / V tiles there; inside a group of LF_BW_GROUP pairs the long q tiles come first.
  const int nrow = (p.Hq / p.Hkv) * nqt;                  // (query head of the group, q tile) per pair
  const int slot = blockIdx.x / 8;
  const int in_grp = slot % (LF_BW_GROUP * nrow);
  const int row = in_grp / LF_BW_GROUP;
  const int bhkv = (slot / (LF_BW_GROUP * nrow) * LF_BW_GROUP + in_grp % LF_BW_GROUP) * 8 + (int)(blockIdx.x % 8);
  if (bhkv >= p.B * p.Hkv) return;
  const int qt = nqt - 1 - row / (p.Hq / p.Hkv);
  const int hkv = bhkv % p.Hkv;
  const int b = bhkv / p.Hkv;
  const int h = hkv * (p.Hq / p.Hkv) + row % (p.Hq / p.Hkv);
  const int q0 = kBM * qt;
  const int wq0 = q0 + 32 * wave;
  const int my_q = wq0 + l32;
  const int qr = min(my_q, p.Sq - 1);
  const int nkt = (p.Sk + 63) / 64;

  lf_u32x4 qf[LF_NKS], gf[LF_NKS];
  {
    const lf_elem* qrow = p.q + (long long)b * p.q_sb + (long long)h * p.q_sh + (long long)qr * p.q_ss;
    const lf_elem* grow = p.dout + (long long)b * p.do_sb + (long long)h * p.do_sh + (long long)qr * p.do_ss;
#pragma unroll
    for (int ks = 0; ks < LF_NKS; ++ks) {
      qf[ks] = *reinterpret_cast<const lf_u32x4*>(qrow + 16 * ks + 8 * g);
      gf[ks] = *reinterpret_cast<const lf_u32x4*>(grow + 16 * ks + 8 * g);
    }
#if LF_BW_DQ_ASM
#pragma unroll
    for (int ks = 0; ks < LF_NKS; ++ks) asm volatile("" : "+a"(qf[ks]), "+a"(gf[ks]));
#endif
  }
  const long long ridx = ((long long)b * p.Hq + h) * p.Sq + qr;
  const float lse_q = my_q < p.Sq ? p.lse[ridx] : __builtin_inff();
  const float delta_q = my_q < p.Sq ? p.delta[ridx] : 0.0f;
#if LF_SOFTCAP
  const float sc_exp = p.scale / p.softcap * (2.0f * LF_LOG2E);   // 2^(s * sc_exp) = e^(2x)
  const float cexp = p.softcap * LF_LOG2E;                        // exponent of P: tanh x * cexp - L
#else
  const float cexp = p.scale * LF_LOG2E;
#endif

  lf_f32x16 dq[LF_NDB];
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db) {
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[db][i] = 0.0f;
#if LF_BW_DQ_ASM
    asm volatile("" : "+a"(dq[db]));
#endif
  }

  int kt_begin = 0, kt_end = nkt;
  {
    const int qlast = min(q0 + kBM, p.Sq) - 1;
#if LF_MASK >= 1
    kt_end = min(nkt, qlast / 64 + 1);
#endif
#if LF_MASK == 2
    const int lo = q0 - p.window + 1;
    if (lo > 0) kt_begin = lo / 64;
#endif
    (void)qlast;
  }
  const lf_elem* kbase = p.k + (long long)b * p.k_sb + (long long)hkv * p.k_sh;
  const lf_elem* vbase = p.v + (long long)b * p.v_sb + (long long)hkv * p.v_sh;
  const lf_u32x4 k_rs = lf_make_buffer(kbase, (unsigned)(((long long)(p.Sk - 1) * p.k_ss + LF_D) * 2));
  const lf_u32x4 v_rs = lf_make_buffer(vbase, (unsigned)(((long long)(p.Sk - 1) * p.v_ss + LF_D) * 2));
  // the direct loads of tile kt + 1 go out one by one behind MFMA pairs of the first products of
  // tile kt (a wave owes 3 * kPasses per tile); past the last tile they go out against an empty
  // range and fetch nothing
  constexpr int kPasses = 64 * LF_CPR / LF_BW_DQ_NT;
  constexpr int kLoads = 3 * kPasses;
  static_assert(kLoads <= 2 * LF_NKS, "one direct load per pair of MFMAs of the first products");
  lf_u32x4 k_cur = k_rs, v_cur = v_rs;
  const unsigned lane_off[3] = {lf_bw_dma_lane_off<LF_BW_DQ_NT>((unsigned)p.k_ss * 2u, false, tid),
                                lf_bw_dma_lane_off<LF_BW_DQ_NT>((unsigned)p.k_ss * 2u, true, tid),
                                lf_bw_dma_lane_off<LF_BW_DQ_NT>((unsigned)p.v_ss * 2u, false, tid)};
  auto issue_piece = [&](int kt, int st, int j) {      // tile j / kPasses (K, K transposed, V), pass j % kPasses
    const int t = j / kPasses;
    lf_bw_dma_piece<LF_BW_DQ_NT>(t < 2 ? k_cur : v_cur, (unsigned)(t < 2 ? p.k_ss : p.v_ss) * 2u, 64 * kt, tiles[st][t],
                                 lane_off[t], j % kPasses, wave);
  };
  if (kt_begin < kt_end) {
#pragma unroll
    for (int j = 0; j < kLoads; ++j) issue_piece(kt_begin, 0, j);
  }
  LF_BW_BARRIER();
  for (int kt = kt_begin; kt < kt_end; ++kt) {
    const int k0 = 64 * kt;
    const int st = (kt - kt_begin) & 1;
    const lf_elem* k_rm = tiles[st][0];
    const lf_elem* k_tr = tiles[st][1];
    const lf_elem* v_rm = tiles[st][2];
    if (kt + 1 >= kt_end) k_cur[2] = v_cur[2] = 0u;   // the other stage is free: every wave left it at the last barrier
#if !LF_BW_DQ_ASM      // 8 waves: a wave owes few loads and has no registers to spare for their offsets
#pragma unroll
    for (int j = 0; j < kLoads; ++j) issue_piece(kt + 1, st ^ 1, j);
#endif

    bool need = wq0 < p.Sq;
#if LF_MASK >= 1
    need = need && (k0 <= min(wq0 + 31, p.Sq - 1));
#endif
#if LF_MASK == 2
    need = need && (min(k0 + 64, p.Sk) - 1 >= wq0 - p.window + 1);
#endif
    if (need) {
    // are all 64 x 32 scores of this wave kept?  Then the tile runs without the mask arithmetic
    bool full = k0 + 63 < p.Sk;
#if LF_MASK >= 1
    full = full && (k0 + 63 <= wq0);
#endif
#if LF_MASK == 2
    full = full && (wq0 + 31 - k0 < p.window);
#endif
    const bool masked = !full;

    lf_u32x4 dsf[LF_NKK];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      lf_f32x16 s, dp;
      lf_u32x4 ka[LF_NKS], va[LF_NKS];
#pragma unroll
      for (int ks = 0; ks < LF_BW_DQ_PF1; ++ks) {
        ka[ks] = lf_read_k_frag(k_rm, l32, g, ks * LF_NKB + kb);
        va[ks] = lf_read_k_frag(v_rm, l32, g, ks * LF_NKB + kb);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < LF_NKS; ++ks) {
        if (ks + LF_BW_DQ_PF1 < LF_NKS) {
          ka[ks + LF_BW_DQ_PF1] = lf_read_k_frag(k_rm, l32, g, (ks + LF_BW_DQ_PF1) * LF_NKB + kb);
          va[ks + LF_BW_DQ_PF1] = lf_read_k_frag(v_rm, l32, g, (ks + LF_BW_DQ_PF1) * LF_NKB + kb);
        }
        lf_bw_dq_mfma_s(s, ka[ks], qf[ks], ks == 0);         // S^T[key][q]
        lf_bw_dq_mfma_s(dp, va[ks], gf[ks], ks == 0);        // dP^T[key][q]
#if LF_BW_DQ_ASM
        if (LF_NKS * kb + ks < kLoads) issue_piece(kt + 1, st ^ 1, LF_NKS * kb + ks);
#endif
        __builtin_amdgcn_sched_barrier(0);
      }
#if LF_BW_DQ_ASM
      asm volatile(LF_BW_MFMA_DRAIN : "+v"(s), "+v"(dp));
#endif
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        lf_elem4 dw;
        float pv[4];
#if LF_SOFTCAP
        float dcap[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float r = __builtin_amdgcn_rcpf(1.0f + lf_exp2(s[4 * i4 + e] * sc_exp));
          pv[e] = lf_exp2((1.0f - 2.0f * r) * cexp - lse_q);
          dcap[e] = 4.0f * r * (1.0f - r);
        }
#else
#pragma unroll
        for (int e = 0; e < 4; ++e) pv[e] = lf_exp2(s[4 * i4 + e] * cexp - lse_q);
#endif
        if (masked) {           // wave-uniform: most tiles of a q tile lie below the diagonal
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int j = k0 + 32 * kb + 8 * i4 + 4 * g + e;
            pv[e] = (j < p.Sk && lf_bw_keep(my_q - j, p.window)) ? pv[e] : 0.0f;
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#if LF_SOFTCAP
          dw[e] = lf_from_float(pv[e] * (dp[4 * i4 + e] - delta_q) * dcap[e]);
#else
          dw[e] = lf_from_float(pv[e] * (dp[4 * i4 + e] - delta_q));   // dS without `scale`
#endif
        }
        const lf_u32x2 du = __builtin_bit_cast(lf_u32x2, dw);
        dsf[2 * kb + i4 / 2][2 * (i4 % 2)] = du[0];
        dsf[2 * kb + i4 / 2][2 * (i4 % 2) + 1] = du[1];
      }
    }
    // dQ^T += K^T dS^T (k = the 64 keys of the tile)
    {
      constexpr int kNF = LF_NKK * LF_NDB;
      lf_u32x4 kt2[kNF];
      // the addresses of the transposed reads are formed again in every step: held across the
      // first products they do not fit the 256 registers of a wave and end up in scratch memory
      int lane_r = lane;
      asm volatile("" : "+v"(lane_r));
      const int g_r = lane_r >> 5;
#pragma unroll
      for (int f = 0; f < LF_BW_PF2; ++f) kt2[f] = __builtin_bit_cast(lf_u32x4, lf_read_v_frag_tr(k_tr, lane_r, g_r, f));
      __builtin_amdgcn_sched_barrier(0);
#if LF_BW_DQ_ASM
#pragma unroll
      for (int kk = 0; kk < LF_NKK; ++kk) asm volatile(LF_BW_VALU_SETTLE : "+v"(dsf[kk]));
#endif
#pragma unroll
      for (int f = 0; f < kNF; ++f) {
        if (f + LF_BW_PF2 < kNF) kt2[f + LF_BW_PF2] = __builtin_bit_cast(lf_u32x4, lf_read_v_frag_tr(k_tr, lane_r, g_r, f + LF_BW_PF2));
        lf_bw_dq_mfma_acc(dq[f % LF_NDB], kt2[f], dsf[f / LF_NDB]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    } else {
#if LF_BW_DQ_ASM
#pragma unroll
      for (int j = 0; j < kLoads; ++j) issue_piece(kt + 1, st ^ 1, j);
#endif
    }
    LF_BW_BARRIER();
  }
#if LF_BW_DQ_ASM
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db) asm volatile(LF_BW_MFMA_DRAIN_LAST : "+a"(dq[db]));
#endif
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[db][i] *= p.scale;
  lf_bw_store_rows(dq, p.dq + (long long)b * p.dq_sb + (long long)h * p.dq_sh + (long long)qr * p.dq_ss, my_q < p.Sq, g);
}
