// lf_attn_prefill.hip — fused attention forward for gfx950 (prefill shapes).
//
// One workgroup = LF_NW waves x 32 query rows; it walks the KV sequence in
// tiles of LF_BN rows that are staged (double-buffered, XOR-swizzled) in LDS.
// Per KV tile each wave computes, entirely in registers,
//     S^T = K Q^T          (v_mfma_f32_32x32x16, K fragment from LDS, Q in VGPRs)
//     score mods + mask    (scale / softcap / causal / window / bounds)
//     online softmax       (lane-local over the 16*LF_BN/32 scores a lane owns,
//                           one exchange with lane^32)
//     O^T += V^T P^T       (V fragment read transposed from LDS)
// Working on the transposed problem makes the accumulator layout of S^T equal to
// the B-operand layout of the second product, so P never leaves registers, and
// makes every per-query quantity (running max, sum, rescale factor) a per-lane
// scalar.  This is the loop nest the reference's optimiser derives for attention
// (loopfuse/compiler/passes/factor_acc.py:23-109 for the rescaled accumulation,
// loopfuse/compiler/passes/skip_loop_iterations.py:343-376 for the tile bounds)
// and hands to its Triton emitter (loopfuse/codegen.py:699-712).
//
// Extra compile-time switches:
//   LF_V_TR   1: read V fragments with ds_read_b64_tr_b16; 0: scalar LDS reads

#ifndef LF_V_TR
#define LF_V_TR 1
#endif
#ifndef LF_SETPRIO
#define LF_SETPRIO 1     /* raise wave priority while it issues MFMAs */
#endif
#ifndef LF_KPF
#define LF_KPF 6         /* K fragments in flight ahead of the MFMA consuming them */
#endif
#ifndef LF_VPF
#define LF_VPF 4         /* V fragments (two transposed reads each) in flight */
#endif
#ifndef LF_KVBUF
#define LF_KVBUF 1       /* dense K/V staged with range-checked buffer loads (needs < 2 GiB per (batch, head) span) */
#endif
#ifndef LF_DMA
#define LF_DMA 0   /* 1 (needs LF_KVBUF): dense K/V tiles go global -> LDS directly (buffer_load ... lds
                      through inline asm), which frees the staging registers; used where the kernel
                      needs them for bias values or the second score product */
#endif
#if LF_DMA > 1
#error "LF_DMA is 0 or 1"
#endif
#define LF_DMA_K (LF_DMA && !(LF_PAGED & 1))
#define LF_DMA_V (LF_DMA && !(LF_PAGED & 2))
#ifndef LF_LAZY_LOG2
#define LF_LAZY_LOG2 8   /* slack of the softmax exponent offset, log2 units */
#endif

#ifndef LF_D2
#define LF_D2 0     /* depth of a second score product: S = Q K^T + Q2 K2^T (16, 32 or 64; 0 = none) */
#endif

#ifndef LF_OCC
#define LF_OCC 2    /* waves per SIMD the register budget is set for */
#endif
#ifndef LF_NW
#define LF_NW 4     /* waves per workgroup (4 or 8) */
#endif
#define LF_NT (LF_NW * 64)
#define LF_BM (32 * LF_NW)
#define LF_NPASS (LF_BN * LF_CPR / LF_NT)    /* staging passes per tile       */
#define LF_CPR2 (LF_D2 / 8)                  /* 16-byte chunks per K2 row      */
#define LF_NKS2 (LF_D2 / 16)                 /* k-steps of the Q2 K2^T product */
#define LF_RPS2 (LF_D2 ? 256 / (LF_D2 * 2) : 1)
#define LF_NP2 ((LF_BN * LF_CPR2 + LF_NT - 1) / LF_NT)   /* staging passes of a K2 tile */
// LDS row strides (elements): rows are not padded, the tiles are XOR-swizzled
#define LF_KS LF_D
#define LF_VS LF_D

#if LF_D2
// The K2 tile (rows of LF_D2 elements, several rows per 256-byte bank span): the K tile's
// permutation (lf_k_phys) with its own row length.
__device__ __forceinline__ int lf_k2_phys(int row, int ch) {
  return ch ^ ((row / LF_RPS2) & (LF_CPR2 - 1));
}
#endif


// Mask tensors reach the kernel as score biases of 0 / -inf.  Before the loop over a q
// tile's KV tiles the workgroup looks for tiles whose bias is -inf for all of its rows and
// keys: they add nothing (every probability is 0) and the loop leaves them out, loads
// included.  Needs 8-byte aligned bias rows; not combined with the second score product
// (no LDS left for the list at two workgroups per CU).
#ifndef LF_BIAS_EARLY
/* request a tile's bias values before its S^T products (not where the registers are short:
   second score product, element-wise loads of unaligned rows) */
#define LF_BIAS_EARLY (!LF_D2 && !(LF_BIAS & 4))
#endif
#ifndef LF_LIVE_LIST
#define LF_LIVE_LIST 1        /* 0: walk every tile (for comparisons) */
#endif
#define LF_USE_LIVE_LIST (LF_LIVE_LIST && (LF_BIAS & 1) && !(LF_BIAS & 4) && !LF_D2)
#define LF_LIVE_WORDS 64      /* 64-bit words of the list: q tiles with up to 4096 KV tiles use it */

extern "C" __global__ void __launch_bounds__(LF_NT, LF_OCC) lf_attn_prefill(const LfAttnParams p) {
  __shared__ __attribute__((aligned(16))) lf_elem lds_k[2][LF_BN * LF_KS];
  __shared__ __attribute__((aligned(16))) lf_elem lds_v[2][LF_BN * LF_VS];
#if LF_USE_LIVE_LIST
  __shared__ unsigned long long lds_dead[LF_LIVE_WORDS];     // bit r of word w: KV tile kt_begin + 64 w + r is dead
  static_assert(sizeof(lf_elem) * LF_BN * LF_VS >= 5 * LF_LIVE_WORDS * sizeof(unsigned long long),
                "the second V buffer holds the scratch of the dead-tile search");
#endif
#if LF_D2
  __shared__ __attribute__((aligned(16))) lf_elem lds_k2[2][LF_BN * LF_D2];
#endif

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // ---- workgroup -> (batch*head, q tile).  Workgroup ids are dealt round-robin
  // to the 8 XCDs, so ids with equal id%8 share an L2: keep all q tiles of one
  // (batch, head) on one XCD, heaviest (latest) q tile first.
  const int nqt = (p.Sq + LF_BM - 1) / LF_BM;
  const int npair = (nqt + 1) / 2;
  const int nbh = p.B * p.Hq;
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  // within an XCD: groups of 4 (batch, head) pairs (their K/V fit the 4 MB L2
  // together); a workgroup takes q tile nqt-1-i and then q tile i of its (batch,
  // head), so that under a causal mask every workgroup walks the same number of
  // KV tiles (2(i+1) + 2(nqt-i) of them) and the grid has no long tail
  const int grp = slot / (4 * npair);
  const int in_grp = slot % (4 * npair);
  const int bh = (grp * 4 + (in_grp & 3)) * 8 + xcd;
  if (bh >= nbh) return;
  const int pair = in_grp >> 2;
  const int b = bh / p.Hq;
  const int h = bh % p.Hq;
  const int hkv = h / (p.Hq / p.Hkv);
  const int nkt = (p.Sk + LF_BN - 1) / LF_BN;

  auto run_q_tile = [&](const int qt) {
  const int q0 = qt * LF_BM;
  const int qlast = min(q0 + LF_BM, p.Sq) - 1;

  // ---- block skip: KV tiles [kt_begin, kt_end) are those with at least one
  // unmasked (i, j) for rows q0..qlast.
  int kt_begin = 0, kt_end = nkt;
#if LF_MASK >= 1
  kt_end = min(nkt, qlast / LF_BN + 1);
#endif
#if LF_MASK == 2
  {
    int lo = q0 - p.window + 1;
    if (lo > 0) kt_begin = lo / LF_BN;
  }
#endif
  if (p.visits != nullptr && tid == 0) {
    for (int kt = kt_begin; kt < kt_end; ++kt)
      p.visits[((long long)bh * nqt + qt) * nkt + kt] = 1;
  }

  // ---- this wave's rows
  const int wq0 = q0 + 32 * wave;
  const int wqlast = min(wq0 + 31, p.Sq - 1);
  const bool wave_has_rows = wq0 < p.Sq;
  const int my_q = wq0 + l32;

  // Q^T fragments (B operand): lane holds row my_q, d = 16*ks + 8*g .. +7.
  lf_elem8 qf[LF_NKS];
  {
    const lf_elem* qrow = p.q + (long long)b * p.q_sb + (long long)h * p.q_sh + (long long)my_q * p.q_ss;
#pragma unroll
    for (int ks = 0; ks < LF_NKS; ++ks) {
      lf_u32x4 raw = {0u, 0u, 0u, 0u};
      if (my_q < p.Sq) raw = *reinterpret_cast<const lf_u32x4*>(qrow + 16 * ks + 8 * g);
      qf[ks] = __builtin_bit_cast(lf_elem8, raw);
    }
  }

#if LF_D2
  lf_elem8 qf2[LF_NKS2];
  {
    const lf_elem* qrow = p.q2 + (long long)b * p.q2_sb + (long long)h * p.q2_sh + (long long)my_q * p.q2_ss;
#pragma unroll
    for (int ks = 0; ks < LF_NKS2; ++ks) {
      lf_u32x4 raw = {0u, 0u, 0u, 0u};
      if (my_q < p.Sq) raw = *reinterpret_cast<const lf_u32x4*>(qrow + 16 * ks + 8 * g);
      qf2[ks] = __builtin_bit_cast(lf_elem8, raw);
    }
  }
  // K2 tile: plain loads with the row clamped to Sk-1 (scores of rows past Sk are masked)
  lf_u32x4 k2st[LF_NP2];
  const lf_elem* k2_uni = p.k2 + (long long)b * p.k2_sb + (long long)(h / p.k2_group) * p.k2_sh;
#endif

#if LF_SOFTCAP && !(LF_BIAS & 1)
  // capped score c*tanh(x) = c - 2c*r with r = 1 / (e^(2x) + 1), x = s*scale/c.  The
  // constant c is the same for every key of a row, so the softmax does not see it: the
  // kernel works on -r and folds the factor 2c into the exponent multiplier
  const float sc_exp = p.scale / p.softcap * (2.0f * LF_LOG2E);   // 2^(s * sc_exp) = e^(2x)
  const float cexp = 2.0f * p.softcap * LF_LOG2E;
#elif LF_SOFTCAP
  const float sc_in = p.scale / p.softcap;   // tanh argument multiplier
  const float cexp = LF_LOG2E;               // scores are final before exp (a bias is added to them)
#elif LF_BIAS & 1
  const float cexp = LF_LOG2E;               // scores are scaled explicitly, then biased
#else
  const float cexp = p.scale * LF_LOG2E;     // scale folded into the exponent
#endif

  lf_f32x16 o[LF_NDB];
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.0f;
  float mc_ref = LF_NEG_INF;  // exponent offset of this query in log2 units (a lagging running max)
#if LF_DENOM
  float mc_true = LF_NEG_INF; // the running max itself (the extra denominator term is relative to it)
#endif
  float l_run = 0.0f;         // this lane's share of the running sum

  // ---- staging: thread handles chunk (srow + kRowsPerPass*ps, sch) of every pass.
  // Dense K/V go through buffer loads: one resource per tensor covering rows
  // 0..Sk-1 of this (batch, kv head); the byte offset (a fixed per-thread part plus
  // a uniform tile/pass part) is range-checked by the hardware, so rows past Sk read
  // as zeros (their scores are masked, their probabilities exactly 0) and the loop
  // carries one 32-bit add per load instead of 64-bit address arithmetic.
  // Paged K/V: plain global loads through the page table, rows clamped to Sk-1.
  lf_u32x4 kst[LF_NPASS], vst[LF_NPASS];
  constexpr int kRowsPerPass = LF_NT / LF_CPR;
  const int srow = tid / LF_CPR;
  const int sch = tid % LF_CPR;
  const lf_elem* k_uni = p.k + (long long)b * p.k_sb + (long long)hkv * p.k_sh;
  const lf_elem* v_uni = p.v + (long long)b * p.v_sb + (long long)hkv * p.v_sh;
#if LF_KVBUF
  const unsigned k_bytes = (unsigned)(((long long)(p.Sk - 1) * p.k_ss + LF_D) * 2);
  const unsigned v_bytes = (unsigned)(((long long)(p.Sk - 1) * p.v_ss + LF_D) * 2);
  const __amdgpu_buffer_rsrc_t k_rs = __builtin_amdgcn_make_buffer_rsrc((void*)k_uni, 0, (int)k_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc((void*)v_uni, 0, (int)v_bytes, 0x00020000);
  const unsigned k_toff = ((unsigned)(srow * p.k_ss) + 8u * sch) * 2u;      // bytes
  const unsigned v_toff = ((unsigned)(srow * p.v_ss) + 8u * sch) * 2u;
  const unsigned k_rowb = (unsigned)p.k_ss * 2u, v_rowb = (unsigned)p.v_ss * 2u;
#endif
#if LF_DMA
  // Direct global -> LDS staging: a wave-level buffer_load_dwordx4 ... lds writes
  // 64 lanes x 16 B to LDS at M0 + 16*lane, i.e. 64/LF_CPR whole rows of the
  // (unpadded, row-major) tile; the XOR swizzle is applied on the global side: the
  // lane that lands on physical chunk `sch` fetches logical chunk sch ^ swizzle(row).
  // No staging registers, no ds_write, and rows past Sk arrive as zeros.
  const lf_u32x4 k_rsq = lf_make_buffer(k_uni, k_bytes), v_rsq = lf_make_buffer(v_uni, v_bytes);
  const unsigned k_doff = (unsigned)srow * k_rowb + 16u * (unsigned)lf_k_phys(srow, sch);
  const unsigned v_doff = (unsigned)srow * v_rowb + 16u * (unsigned)lf_v_phys(srow, sch);
  constexpr int kRowsPerWave = 64 / LF_CPR;
  auto dma = [&](const lf_u32x4& rs, unsigned voff, const lf_elem* lds_row0) { lf_dma_to_lds(rs, voff, lds_row0); };
#endif
  auto load_tile = [&](int kt, int buf) {
#pragma unroll
    for (int ps = 0; ps < LF_NPASS; ++ps) {
      const int r0 = kt * LF_BN + kRowsPerPass * ps;    // uniform
      (void)buf;
#if LF_DMA_K
      dma(k_rsq, k_doff + (unsigned)r0 * k_rowb, &lds_k[buf][(kRowsPerPass * ps + kRowsPerWave * wave) * LF_KS]);
#else
      if ((LF_PAGED & 1) || !LF_KVBUF) {
        const int tok = min(r0 + srow, p.Sk - 1);
        kst[ps] = *reinterpret_cast<const lf_u32x4*>(lf_kv_row(p, 0, b, hkv, tok) + 8 * sch);
      } else {
#if LF_KVBUF
        kst[ps] = __builtin_amdgcn_raw_buffer_load_b128(k_rs, k_toff + (unsigned)r0 * k_rowb, 0, 0);
#endif
      }
#endif
#if LF_DMA_V
      dma(v_rsq, v_doff + (unsigned)r0 * v_rowb, &lds_v[buf][(kRowsPerPass * ps + kRowsPerWave * wave) * LF_VS]);
#else
      if ((LF_PAGED & 2) || !LF_KVBUF) {
        const int tok = min(r0 + srow, p.Sk - 1);
        vst[ps] = *reinterpret_cast<const lf_u32x4*>(lf_kv_row(p, 1, b, hkv, tok) + 8 * sch);
      } else {
#if LF_KVBUF
        vst[ps] = __builtin_amdgcn_raw_buffer_load_b128(v_rs, v_toff + (unsigned)r0 * v_rowb, 0, 0);
#endif
      }
#endif
    }
#if LF_D2
#pragma unroll
    for (int ps = 0; ps < LF_NP2; ++ps) {
      const int c = tid + LF_NT * ps;
      if (c < LF_BN * LF_CPR2) {
        const int tok = min(kt * LF_BN + c / LF_CPR2, p.Sk - 1);
        k2st[ps] = *reinterpret_cast<const lf_u32x4*>(k2_uni + (long long)tok * p.k2_ss + 8 * (c % LF_CPR2));
      }
    }
#endif
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int ps = 0; ps < LF_NPASS; ++ps) {
      const int row = srow + kRowsPerPass * ps;
      (void)row;
#if !LF_DMA_K
      *reinterpret_cast<lf_u32x4*>(&lds_k[buf][row * LF_KS + 8 * lf_k_phys(row, sch)]) = kst[ps];
#endif
#if !LF_DMA_V
      *reinterpret_cast<lf_u32x4*>(&lds_v[buf][row * LF_VS + 8 * lf_v_phys(row, sch)]) = vst[ps];
#endif
    }
#if LF_D2
#pragma unroll
    for (int ps = 0; ps < LF_NP2; ++ps) {
      const int c = tid + LF_NT * ps;
      if (c < LF_BN * LF_CPR2) {
        const int row = c / LF_CPR2;
        *reinterpret_cast<lf_u32x4*>(&lds_k2[buf][row * LF_D2 + 8 * lf_k2_phys(row, c % LF_CPR2)]) = k2st[ps];
      }
    }
#endif
#if LF_DMA_K || LF_DMA_V
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's direct-to-LDS loads have landed
#endif
  };

#if LF_USE_LIVE_LIST
  // ---- dead KV tiles of this q tile.  Scratch: the second V buffer, which nothing uses
  // before the loop's first iteration (and the previous q tile's loop ended on a barrier).
  const int nrel = kt_end - kt_begin;
  const bool use_list = nrel <= 64 * LF_LIVE_WORDS;
  if (use_list) {
    unsigned long long* cand = reinterpret_cast<unsigned long long*>(&lds_v[1][0]);      // [LF_LIVE_WORDS]
    unsigned long long* part = cand + LF_LIVE_WORDS;                                      // [LF_NW][LF_LIVE_WORDS]
    const int nwords = (nrel + 63) / 64;
    const lf_elem* bbase = p.bias + (long long)b * p.bias_sb + (long long)h * p.bias_sh;
    // (1) candidates: whole tiles (not the one that crosses Sk) with -inf at the bottom-left
    // and the top-right corner (a dense bias stops here: two loads per tile)
    for (int wi = wave; wi < nwords; wi += LF_NW) {
      const int rel = 64 * wi + lane;
      const int kc = min(kt_begin + rel, kt_end - 1) * LF_BN;        // first key of the tile, < Sk
      const unsigned short bl = __builtin_bit_cast(unsigned short, bbase[(long long)qlast * p.bias_sq + kc]);
      const unsigned short tr = __builtin_bit_cast(unsigned short, bbase[(long long)q0 * p.bias_sq + min(kc + LF_BN, p.Sk) - 1]);
      const unsigned long long word = __builtin_amdgcn_ballot_w64(rel < nrel && kc + LF_BN <= p.Sk &&
                                                                  lf_bias_masked(bl) && lf_bias_masked(tr));
      if (lane == 0) cand[wi] = word;
    }
    __syncthreads();
    // (2) every wave checks its own 32 rows of each candidate, four candidates at a time
    // (their loads are in flight together): lane (l32, g) reads row wq0 + l32 (clamped),
    // keys 32 g .. 32 g + 31 of the tile
    {
      const lf_elem* brow_w = bbase + (long long)min(wq0 + l32, p.Sq - 1) * p.bias_sq + 32 * g;
      for (int wi = 0; wi < nwords; ++wi) {
        const unsigned long long cw = cand[wi];
        const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)cw);
        const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(cw >> 32));
        unsigned long long mine = ((unsigned long long)hi << 32) | lo;
        unsigned long long todo = mine;
        while (todo != 0ull) {
          int bits[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            bits[c] = todo != 0ull ? __builtin_ctzll(todo) : bits[0];     // a repeat of the first is harmless
            todo &= todo - 1ull;                                           // 0 stays 0
          }
          lf_u32x2 raw[4][8];
#pragma unroll
          for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i)
              raw[c][i] = *reinterpret_cast<const lf_u32x2*>(brow_w + (kt_begin + 64 * wi + bits[c]) * LF_BN + 4 * i);
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            bool dead = true;
#pragma unroll
            for (int i = 0; i < 8; ++i) dead = dead && lf_bias_masked2(raw[c][i][0]) && lf_bias_masked2(raw[c][i][1]);
            if (__builtin_amdgcn_ballot_w64(dead) != ~0ull) mine &= ~(1ull << bits[c]);
          }
        }
        if (lane == 0) part[wave * LF_LIVE_WORDS + wi] = mine;
      }
    }
    __syncthreads();
    // (3) dead for the workgroup = dead for each of its waves
    if (tid < nwords) {
      unsigned long long d = part[tid];
#pragma unroll
      for (int w = 1; w < LF_NW; ++w) d &= part[w * LF_LIVE_WORDS + tid];
      lds_dead[tid] = d;
    }
    __syncthreads();
  }
  // first live KV tile at or after kt (kt_end if there is none); wave-uniform
  auto next_live = [&](int kt) -> int {
    if (!use_list) return kt;
    int rel = kt - kt_begin;
    while (rel < nrel) {
      const unsigned long long dw = lds_dead[rel >> 6];
      const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)dw);
      const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(dw >> 32));
      const unsigned long long live = ~(((unsigned long long)hi << 32) | lo) >> (rel & 63);
      if (live != 0ull) {
        rel += __builtin_ctzll(live);
        break;
      }
      rel = (rel | 63) + 1;
    }
    return min(kt_begin + rel, kt_end);
  };

  // the loop walks the live tiles only (all of them can be dead)
  const int kt_first = next_live(kt_begin);
  if (kt_first < kt_end) {
    load_tile(kt_first, 0);
    store_tile(0);
  }
  __syncthreads();

  int cur = 0;
  for (int kt = kt_first, kt_next; kt < kt_end; kt = kt_next, cur ^= 1) {
    kt_next = next_live(kt + 1);
    const bool have_next = kt_next < kt_end;
    if (have_next) load_tile(kt_next, cur ^ 1);
#else
  // every valid q tile has at least one KV tile (kt_end >= 1 > kt_begin is not
  // guaranteed only for Sk == 0, which the host rejects)
  load_tile(kt_begin, 0);
  store_tile(0);
  __syncthreads();

  for (int kt = kt_begin; kt < kt_end; ++kt) {
    const int cur = (kt - kt_begin) & 1;
    const bool have_next = kt + 1 < kt_end;
    if (have_next) load_tile(kt + 1, cur ^ 1);
#endif

    const int k0 = kt * LF_BN;
    bool need = wave_has_rows;
    bool full = (k0 + LF_BN <= p.Sk);
#if LF_MASK >= 1
    need = need && (k0 <= wqlast);
    full = full && (k0 + LF_BN - 1 <= wq0);
#endif
#if LF_MASK == 2
    need = need && (min(k0 + LF_BN, p.Sk) - 1 >= wq0 - p.window + 1);
    full = full && (wq0 + 31 - k0 < p.window);
#endif

    if (need) {
      const lf_elem* kbuf = lds_k[cur];
      const lf_elem* vbuf = lds_v[cur];
#if (LF_BIAS & 1) && LF_BIAS_EARLY
      // the tile's bias values are requested before the S^T products, which hide the latency
      lf_elem4 bias_v[LF_NKB][4];
      {
        const lf_elem* brow = p.bias + (long long)b * p.bias_sb + (long long)h * p.bias_sh +
                              (long long)min(my_q, p.Sq - 1) * p.bias_sq;
#pragma unroll
        for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const int j0 = k0 + 32 * kb + 8 * i4 + 4 * g;
            if (!(LF_BIAS & 4) && j0 + 3 < p.Sk) {
              bias_v[kb][i4] = *reinterpret_cast<const lf_elem4*>(brow + j0);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) bias_v[kb][i4][e] = brow[min(j0 + e, p.Sk - 1)];
            }
          }
      }
#endif

      // ---- S^T = K Q^T (the LF_NKB accumulator chains are interleaved so that
      // consecutive MFMAs are independent)
      lf_f32x16 s[LF_NKB];
#pragma unroll
      for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kb][i] = 0.0f;
#if LF_SETPRIO
      __builtin_amdgcn_s_setprio(2);
#endif
      {
        // K fragments are fetched LF_KPF MFMAs ahead of their use: the LDS round
        // trip (well over 100 cycles) spans several 32-cycle MFMAs
        constexpr int kNF = (LF_NKS * LF_NKB);
        lf_u32x4 kf[kNF > 0 ? kNF : 1];
        auto k_frag = [&](int f) { return lf_read_k_frag(kbuf, l32, g, f); };
#pragma unroll
        for (int f = 0; f < LF_KPF && f < kNF; ++f) kf[f] = k_frag(f);
#pragma unroll
        for (int f = 0; f < kNF; ++f) {
          if (f + LF_KPF < kNF) kf[f + LF_KPF] = k_frag(f + LF_KPF);
          s[f % LF_NKB] = lf_mfma32(__builtin_bit_cast(lf_elem8, kf[f]), qf[f / LF_NKB], s[f % LF_NKB]);
        }
#if LF_D2
        // + Q2 K2^T into the same accumulators
        {
          const lf_elem* k2buf = lds_k2[cur];
#pragma unroll
          for (int f = 0; f < LF_NKS2 * LF_NKB; ++f) {
            const int ks = f / LF_NKB, kb = f % LF_NKB;
            const int row = 32 * kb + l32;
            const lf_u32x4 kv = *reinterpret_cast<const lf_u32x4*>(&k2buf[row * LF_D2 + 8 * lf_k2_phys(row, 2 * ks + g)]);
            s[kb] = lf_mfma32(__builtin_bit_cast(lf_elem8, kv), qf2[ks], s[kb]);
          }
        }
#endif
      }
#if LF_SETPRIO
      __builtin_amdgcn_s_setprio(0);
#endif

      // ---- score modifications and mask; element i of block kb is kv index
      // j = k0 + 32*kb + 8*(i/4) + 4*g + i%4, query my_q.
#if LF_SOFTCAP && !(LF_BIAS & 1)
#pragma unroll
      for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kb][i] = __builtin_amdgcn_rcpf(-1.0f - lf_exp2(s[kb][i] * sc_exp));   // -r
#elif LF_SOFTCAP
#pragma unroll
      for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kb][i] = p.softcap * lf_tanh(s[kb][i] * sc_in);
#endif
#if LF_BIAS & 1
      // additive score bias (reference tests/test_accuracy.py:172-196 "modified attention"):
      // x = scale * s (or the capped score) + bias[b, h, my_q, j]; four consecutive keys
      // per 8-byte load, element-wise with clamped indices where the group crosses Sk
      {
        const lf_elem* brow = p.bias + (long long)b * p.bias_sb + (long long)h * p.bias_sh +
                              (long long)min(my_q, p.Sq - 1) * p.bias_sq;
#pragma unroll
        for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const int j0 = k0 + 32 * kb + 8 * i4 + 4 * g;
            lf_elem4 bv;
#if LF_BIAS_EARLY
            (void)j0;
            (void)brow;
            bv = bias_v[kb][i4];
#else
            if (!(LF_BIAS & 4) && j0 + 3 < p.Sk) {
              bv = *reinterpret_cast<const lf_elem4*>(brow + j0);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) bv[e] = brow[min(j0 + e, p.Sk - 1)];
            }
#endif
#pragma unroll
            for (int e = 0; e < 4; ++e) {
#if LF_SOFTCAP
              s[kb][4 * i4 + e] += lf_bias_value(bv[e]);
#else
              s[kb][4 * i4 + e] = s[kb][4 * i4 + e] * p.scale + lf_bias_value(bv[e]);
#endif
            }
          }
      }
#endif
      if (!full) {
#pragma unroll
        for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            int j = k0 + 32 * kb + 8 * (i / 4) + 4 * g + (i % 4);
            bool ok = j < p.Sk;
#if LF_MASK >= 1
            ok = ok && (j <= my_q);
#endif
#if LF_MASK == 2
            ok = ok && (my_q - j < p.window);
#endif
            s[kb][i] = ok ? s[kb][i] : LF_NEG_INF;
          }
      }

      // ---- online softmax (per query = per lane pair l, l^32).  The exponent
      // offset m_ref is allowed to lag behind the true running max by up to
      // LF_LAZY_LOG2 (in log2 units): probabilities then reach at most
      // 2^LF_LAZY_LOG2, which fp32 sums and bf16/fp16 operands hold without loss,
      // and O and l are rescaled only when some query of the wave exceeds the
      // slack -- a wave-uniform branch that is rarely taken after the first tiles.
      // O / l is independent of the offset, so the result is unchanged.
      float mx = LF_NEG_INF;
#pragma unroll
      for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kb][i]);
      mx = fmaxf(mx, lf_swap32(mx));
      const float mxc = mx * cexp;
#if LF_DENOM
      mc_true = fmaxf(mc_true, mxc);
#endif
      if (__builtin_amdgcn_ballot_w64(mxc > mc_ref + (float)LF_LAZY_LOG2) != 0ull) {
        const float mc_new = fmaxf(mc_ref, mxc);          // finite wherever mxc is
        // 0 on a query's first update (its O and l are still 0); 1 for a query
        // that still has seen nothing (both offsets -inf)
        const float r = (mc_new == LF_NEG_INF) ? 1.0f : lf_exp2(mc_ref - mc_new);
        mc_ref = mc_new;
        l_run *= r;
#pragma unroll
        for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[db][i] *= r;
      }
      // a query that has seen no unmasked key yet (offset still -inf) subtracts 0
      const float mc_sub = (mc_ref == LF_NEG_INF) ? 0.0f : mc_ref;

      float rs = 0.0f;
      lf_elem8 pf[LF_NKK];
#pragma unroll
      for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float e = lf_exp2(s[kb][i] * cexp - mc_sub);
          rs += e;
          pf[2 * kb + i / 8][i % 8] = lf_from_float(e);
        }
      l_run += rs;

#if LF_SETPRIO
      __builtin_amdgcn_s_setprio(2);
#endif
      // ---- O^T += V^T P^T.  k-slot s of step kk is kv row
      // 16*kk + 8*(s/4) + 4*g + s%4 (the order P is held in); A row = d.
      {
        constexpr int kNF = (LF_NKK * LF_NDB);
        lf_elem8 vf[kNF > 0 ? kNF : 1];
        auto v_frag = [&](int f) {
          const int kk = f / LF_NDB, db = f % LF_NDB;
          lf_elem8 a;
#if LF_V_TR
          (void)kk;
          (void)db;
          a = lf_read_v_frag_tr(vbuf, lane, g, f);
#else
          const int col = 32 * db + l32;
#pragma unroll
          for (int sl = 0; sl < 8; ++sl) {
            const int row = 16 * kk + 8 * (sl / 4) + 4 * g + (sl % 4);
            a[sl] = vbuf[row * LF_VS + 8 * lf_v_phys(row, col / 8) + (col % 8)];
          }
#endif
          return a;
        };
#pragma unroll
        for (int f = 0; f < LF_VPF && f < kNF; ++f) vf[f] = v_frag(f);
#pragma unroll
        for (int f = 0; f < kNF; ++f) {
          if (f + LF_VPF < kNF) vf[f + LF_VPF] = v_frag(f + LF_VPF);
          o[f % LF_NDB] = lf_mfma32(vf[f], pf[f / LF_NDB], o[f % LF_NDB]);
        }
      }
#if LF_SETPRIO
      __builtin_amdgcn_s_setprio(0);
#endif
    }

    if (have_next) store_tile(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue: O[q][d] = O^T[d][q] / l.  Element i of block db is
  // d = 32*db + 8*(i/4) + 4*g + i%4.
  if (my_q < p.Sq) {
    float l_tot = l_run + lf_swap32(l_run);
#if LF_DENOM
    // sum and extra term in the same units: l is relative to the lagging offset
    l_tot += p.denom_add * lf_exp2(mc_true - mc_ref);
#endif
    const float inv = lf_inv_sum(l_tot);
    lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)h * p.o_sh + (long long)my_q * p.o_ss;
#pragma unroll
    for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        lf_elem4 w;
#if LF_BIAS & 2
        const lf_elem* obp = p.obias + (long long)b * p.ob_sb + (long long)h * p.ob_sh +
                             (long long)my_q * p.ob_sq + 32 * db + 8 * i4 + 4 * g;
        lf_elem4 ob;
        if (LF_BIAS & 4) {
#pragma unroll
          for (int e = 0; e < 4; ++e) ob[e] = obp[e];
        } else {
          ob = *reinterpret_cast<const lf_elem4*>(obp);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = lf_from_float(o[db][4 * i4 + e] * inv + lf_to_float(ob[e]));
#else
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = lf_from_float(o[db][4 * i4 + e] * inv);
#endif
        *reinterpret_cast<lf_elem4*>(orow + 32 * db + 8 * i4 + 4 * g) = w;
      }
  }
  };   // run_q_tile

  run_q_tile(nqt - 1 - pair);
  if (pair != nqt - 1 - pair) run_q_tile(pair);
}
