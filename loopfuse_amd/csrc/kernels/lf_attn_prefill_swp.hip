// lf_attn_prefill_swp.hip — fused attention forward for gfx950 (prefill shapes),
// software-pipelined variant of lf_attn_prefill.hip for dense K/V.
//
// Same math, layouts and operand orders as lf_attn_prefill.hip (4 waves x 32 query
// rows, KV tiles of 64 rows, transposed problem S^T = K Q^T, O^T += V^T P^T,
// XOR-swizzled LDS tiles, transposed V reads, lagging softmax offset, closed-form
// tile bounds; reference loopfuse/compiler/passes/factor_acc.py:23-109,
// loopfuse/compiler/passes/skip_loop_iterations.py:343-376).  What differs is when
// memory operations are issued, so that a wave never waits for a memory round trip
// at the head of an MFMA sequence and never stalls on a burst of loads:
//
//   * K/V tiles go global -> LDS directly (buffer_load_dwordx4 ... lds, range-checked,
//     rows past Sk arrive as zeros).  The loads of K(i+2) and V(i+1) are issued one
//     at a time BETWEEN the MFMAs of S^T(i); no staging registers, no LDS writes.
//   * K lives in three LDS slots, V in two (80 KB, two workgroups per CU): K(i+1) is
//     already resident while tile i is processed, so its first fragments are read
//     during the last MFMAs of O^T(i), across the workgroup barrier.
//   * the first V fragments of tile i are read during the last MFMAs of S^T(i), i.e.
//     before the softmax that separates the two products.
//   * the order of reads, loads and MFMAs is pinned with scheduling barriers.
//
// One workgroup barrier per tile; before it each wave waits for its own direct
// loads (issued a full softmax + product earlier).

#ifndef LF_LAZY_LOG2
#define LF_LAZY_LOG2 8
#endif
#ifndef LF_KPF
#define LF_KPF 6         /* K fragments in flight ahead of the MFMA consuming them */
#endif
#ifndef LF_VPF
#define LF_VPF 4         /* V fragments (two transposed reads each) in flight */
#endif
#ifndef LF_SETPRIO
#define LF_SETPRIO 1     /* raise the wave priority while it issues MFMAs */
#endif
#ifndef LF_NW
#define LF_NW 4     /* waves per workgroup: 4 (two workgroups per CU) or 8 (one) */
#endif
#define LF_NT (LF_NW * 64)
#ifndef LF_GQAPACK
#define LF_GQAPACK 0     /* g = 2 or 4 (grouped-query attention, Hq / Hkv a multiple of g): the waves of a
                            workgroup take the same query rows of g consecutive query heads that share one kv
                            head -- wave w: head w % g, row block w / g -- instead of LF_NW row blocks of one
                            head.  A q tile is then 32 * LF_NW / g rows tall; with g = LF_NW every wave needs
                            exactly the same KV tiles (no wave idles on a tile of the diagonal or of the
                            window's edge), and one K/V tile in LDS serves g heads */
#endif
#if LF_GQAPACK
#define LF_BM (32 * LF_NW / LF_GQAPACK)
#define LF_HEADS_PER_WG LF_GQAPACK
#else
#define LF_BM (32 * LF_NW)
#define LF_HEADS_PER_WG 1
#endif
#define LF_KSLOTS 3
#define LF_VSLOTS 2
#define LF_NPASS (LF_BN * LF_CPR / LF_NT)
#define LF_NFK (LF_NKS * LF_NKB)      /* MFMAs (= K fragments) of S^T per tile */
#define LF_NFV (LF_NKK * LF_NDB)      /* MFMAs (= V fragments) of O^T per tile */
#if LF_KPF > LF_NFK || LF_KPF > LF_NFV || LF_VPF > LF_NFK || LF_VPF > LF_NFV
#error "the fragment read-ahead (LF_KPF, LF_VPF) cannot exceed the fragments of a tile"
#endif
#ifndef LF_WPE
#define LF_WPE (8 / LF_NW)     /* waves per SIMD the register budget is sized for (= workgroups per CU for 4 waves) */
#endif

// workgroup barrier that waits for this wave's direct-to-LDS loads but leaves LDS
// reads in flight (the compiler's own barrier would wait for those too)
#ifndef LF_BIAS
#define LF_BIAS 0        /* 1: additive score bias [B, Hq, Sq, Sk] (a mask given as a tensor) with the tile classes
                            that lf_bias_classify wrote into p.part_acc: dead tiles at either end of a q tile's
                            range are not walked, all-zero tiles cost nothing, the others add their values */
#endif
#define LF_BARRIER_VM0() asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory")

#define LF_CAPPOLY (LF_SOFTCAP && !LF_BIAS)   /* polynomial fast path of the softcap (below) */
#ifndef LF_CAP_TERMS
#define LF_CAP_TERMS 1   /* terms of the polynomial that is fused into the exponent (1 or 2) */
#endif
/* minimax fits of tanh(x)/x - 1 in x^2: one term on |x| <= 0.15 (absolute error of tanh 1.4e-6), two terms on
   |x| <= 0.4 (2.1e-6) */
#define LF_CAP1_X0 0.15f
#define LF_CAP1_B1 (-0.3307545f)
#define LF_CAP2_X0 0.4f
#define LF_CAP2_B1 (-0.33269722f)
#define LF_CAP2_B2 0.12145087f
#ifndef LF_QGROUP
#define LF_QGROUP 8      /* (batch, head) pairs per group of slots */
#endif
#ifndef LF_SPLIT_EXP
#define LF_SPLIT_EXP (!LF_SOFTCAP || !LF_BIAS)     /* second key block's exponentials between the MFMAs of the first (config 2: -0.7 %; no gain with a softcap) */
#endif

extern "C" __global__ void __launch_bounds__(LF_NT, LF_WPE) lf_attn_prefill_swp(const LfAttnParams p) {
  // one array, K slots first
  __shared__ __attribute__((aligned(16))) lf_elem lds_all[(LF_KSLOTS + LF_VSLOTS) * LF_BN * LF_D];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // in a scalar register: what derives from it stays scalar
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // ---- workgroup -> (batch*head, q tile).  blockIdx.x % 8 is the XCD (workgroups go to the
  // XCDs round-robin), so all q tiles of a (batch, head) run on one XCD and share its L2.
  // Within an XCD class the slots come in groups of LF_QGROUP (batch, head) pairs -- so many
  // that the resident workgroups of an XCD walk the K/V of few heads at a time -- and within
  // a group by q tile, the one with the most kv tiles first: workgroups are dispatched in
  // blockIdx order, so under a causal mask the long tiles start early and the short ones
  // fill the end of the launch (longest-first list scheduling).
  const int nqt = (p.Sq + LF_BM - 1) / LF_BM;
  const int nhv = p.Hq / LF_HEADS_PER_WG;     // head units per batch element (heads, or packs of heads)
  const int nbh = p.B * nhv;
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int grp = slot / (LF_QGROUP * nqt);
  const int in_grp = slot % (LF_QGROUP * nqt);
  const int bh = (grp * LF_QGROUP + in_grp % LF_QGROUP) * 8 + xcd;
  if (bh >= nbh) return;     // padding slot of the last group
  const int slot_qt = nqt - 1 - in_grp / LF_QGROUP;
  const int b = bh / nhv;
#if LF_GQAPACK
  const int h = (bh % nhv) * LF_GQAPACK + wave % LF_GQAPACK;    // this wave's query head
#else
  const int h = bh % nhv;
#endif
  const int hkv = h / (p.Hq / p.Hkv);         // the same for all waves: the pack lies inside one group
  const int nkt = (p.Sk + LF_BN - 1) / LF_BN;

  // ---- direct-to-LDS staging: a wave-level load writes 64 lanes x 16 B at
  // M0 + 16*lane, i.e. 64/LF_CPR whole rows of the row-major tile; the XOR swizzle
  // is applied on the global side (the lane that lands on physical chunk c of row r
  // fetches the logical chunk that lives there).
  constexpr int kRowsPerPass = LF_NT / LF_CPR;
  constexpr int kRowsPerWave = 64 / LF_CPR;
  const int srow = tid / LF_CPR;
  const int sch = tid % LF_CPR;
  // Dense K/V: one buffer resource per (batch, kv head), rows 0..Sk-1.  Paged K/V
  // (LF_PAGED, pages of a multiple of 64/LF_CPR tokens, pool < 4 GiB): the resource
  // covers the whole pool, and the uniform part of a load's offset comes from the page
  // table: page id * page stride + head + row inside the page.  The 64/LF_CPR rows of
  // one wave-level load never straddle a page.  Rows past Sk get an offset beyond the
  // resource, so they arrive as zeros in both cases.
  constexpr bool kPagedK = (LF_PAGED & 1) != 0, kPagedV = (LF_PAGED & 2) != 0;
  const lf_elem* k_uni = kPagedK ? p.k : p.k + (long long)b * p.k_sb + (long long)hkv * p.k_sh;
  const lf_elem* v_uni = kPagedV ? p.v : p.v + (long long)b * p.v_sb + (long long)hkv * p.v_sh;
  const unsigned k_bytes = kPagedK ? (unsigned)(p.k_span * 2) : (unsigned)(((long long)(p.Sk - 1) * p.k_ss + LF_D) * 2);
  const unsigned v_bytes = kPagedV ? (unsigned)(p.v_span * 2) : (unsigned)(((long long)(p.Sk - 1) * p.v_ss + LF_D) * 2);
  const unsigned k_rowb = (unsigned)p.k_ss * 2u, v_rowb = (unsigned)p.v_ss * 2u;
  const int wave_u = wave;
  // page id (as a byte offset of the page + this kv head) for the rows of this wave in
  // pass ps of tile kt; tiles / rows past Sk re-use the last page (their rows are zeroed)
  auto page_off = [&](int which, int kt, int ps) -> unsigned {
    const int tok = min(kt * LF_BN + (LF_NT / LF_CPR) * ps + (64 / LF_CPR) * wave_u, p.Sk - 1);
    const lf_table_t* tab = reinterpret_cast<const lf_table_t*>(which ? p.v_table : p.k_table);
    const int psz = which ? LF_PAGE_SIZE_V : LF_PAGE_SIZE;
    const unsigned id = (unsigned)tab[(long long)b * (which ? p.vt_stride : p.kt_stride) + tok / psz];
    return which ? id * (unsigned)(p.v_sb * 2) + (unsigned)hkv * (unsigned)(p.v_sh * 2)
                 : id * (unsigned)(p.k_sb * 2) + (unsigned)hkv * (unsigned)(p.k_sh * 2);
  };
  const lf_u32x4 k_rsq = lf_make_buffer(k_uni, k_bytes), v_rsq = lf_make_buffer(v_uni, v_bytes);
  // per-lane part of the offset: dense = row inside the pass, paged = row inside the wave's load
  const unsigned k_doff = (unsigned)(kPagedK ? srow % (64 / LF_CPR) : srow) * k_rowb + 16u * (unsigned)lf_k_phys(srow, sch);
  const unsigned v_doff = (unsigned)(kPagedV ? srow % (64 / LF_CPR) : srow) * v_rowb + 16u * (unsigned)lf_v_phys(srow, sch);
  // LDS byte addresses of the slots' rows as integers (scalar arithmetic on the constant base)
  const unsigned lds0 = lf_lds_addr(lds_all);
  auto k_row_addr = [&](int sl, int row) { return lds0 + (unsigned)((sl * LF_BN + row) * LF_D * 2); };
  auto v_row_addr = [&](int sl, int row) { return lds0 + (unsigned)(((LF_KSLOTS + sl) * LF_BN + row) * LF_D * 2); };
  // pg: page_off() of the pass (paged operands only; fetched a tile ahead by the caller)
  // `rs`: k_rsq / v_rsq, or the same with an empty range for a tile past the last one (nothing is
  // fetched then; the slot it would fill is free)
  auto dma_k_pass = [&](const lf_u32x4& rs, int kt, int sl, int ps, unsigned pg) {
    unsigned off;
    if (kPagedK) {
      const int tokw = kt * LF_BN + kRowsPerPass * ps + kRowsPerWave * wave_u;     // first row of this wave's load
      off = pg + (unsigned)(tokw % LF_PAGE_SIZE) * k_rowb + k_doff;
      if (tokw + (int)(srow % kRowsPerWave) >= p.Sk) off = 0xffffffffu;
    } else {
      off = k_doff + (unsigned)(kt * LF_BN + kRowsPerPass * ps) * k_rowb;
    }
    lf_dma_to_lds_at(rs, off, k_row_addr(sl, kRowsPerPass * ps + kRowsPerWave * wave_u));
  };
  auto dma_v_pass = [&](const lf_u32x4& rs, int kt, int sl, int ps, unsigned pg) {
    unsigned off;
    if (kPagedV) {
      const int tokw = kt * LF_BN + kRowsPerPass * ps + kRowsPerWave * wave_u;
      off = pg + (unsigned)(tokw % LF_PAGE_SIZE_V) * v_rowb + v_doff;
      if (tokw + (int)(srow % kRowsPerWave) >= p.Sk) off = 0xffffffffu;
    } else {
      off = v_doff + (unsigned)(kt * LF_BN + kRowsPerPass * ps) * v_rowb;
    }
    lf_dma_to_lds_at(rs, off, v_row_addr(sl, kRowsPerPass * ps + kRowsPerWave * wave_u));
  };

#if LF_CAPPOLY
  // Capped score c*tanh(x), x = s*scale/c, in log2 units.  Three forms, chosen per wave and tile (uniformly):
  //  * every score has |x| <= X0 and the tile needs no mask: the cap is an odd polynomial on full-rate FMAs,
  //    evaluated where the exponent is formed, 2^(s*(A0 + A1 s^2 [+ A2 s^4]) - m) -- one transcendental per score
  //    as without a cap (tanh is increasing, so the row maximum is the polynomial of the largest raw score);
  //  * |x| <= 0.4 but beyond X0, or a mask in the way: the two-term polynomial in place, then the plain exponent;
  //  * otherwise c*log2e*(1 - 2r), r = 1 / (e^(2x) + 1), in place (two transcendentals more per score).
  // (derived constants are moved back into scalar registers: uniform float arithmetic is done by the vector
  // ALU, and its results would otherwise occupy a vector register each for the whole kernel)
  auto uni = [](float x) { return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x))); };
  const float cap_a = p.scale / p.softcap;
  const float cap_a2 = cap_a * cap_a;
  const float cap_l2 = uni(p.softcap * LF_LOG2E);
  const float sc_exp = uni(cap_a * (2.0f * LF_LOG2E));            // 2^(s * sc_exp) = e^(2x)
  const float capA0 = uni(p.scale * LF_LOG2E);                    // = c*log2e * a
#if LF_CAP_TERMS >= 2
  const float capA1 = uni(capA0 * cap_a2 * LF_CAP2_B1), capA2 = uni(capA0 * cap_a2 * cap_a2 * LF_CAP2_B2);
  const float cap_smax = uni(LF_CAP2_X0 / fabsf(cap_a));          // |s| up to which the fused polynomial holds
#else
  const float capA1 = uni(capA0 * cap_a2 * LF_CAP1_B1);
  const float cap_smax = uni(LF_CAP1_X0 / fabsf(cap_a));
#endif
  const float capP1 = uni(capA0 * cap_a2 * LF_CAP2_B1), capP2 = uni(capA0 * cap_a2 * cap_a2 * LF_CAP2_B2);
  const float cap_smax2 = uni(LF_CAP2_X0 / fabsf(cap_a));         // ... the in-place polynomial holds
  const float cexp = 1.0f;                                       // scores transformed in place are in log2 units
#elif LF_SOFTCAP
  // with a score bias: capped score c*tanh(x) = c - 2c*r with r = 1 / (e^(2x) + 1), x = s*scale/c.  The
  // constant c is the same for every key of a row, so the softmax does not see it: the
  // kernel works on -r and folds the factor 2c into the exponent multiplier, which saves
  // the three VALU operations per score that would turn r into the capped score
  const float sc_exp = p.scale / p.softcap * (2.0f * LF_LOG2E);   // 2^(s * sc_exp) = e^(2x)
  const float cexp = 2.0f * p.softcap * LF_LOG2E;
#else
  const float cexp = p.scale * LF_LOG2E;
#endif

  // Fragment addresses inside a tile.  The XOR swizzles (lf_k_phys, lf_v_phys) depend on the lane and on
  // which 16-dim step (K) / 32-dim block (V) a fragment belongs to, not on its row block, and the step /
  // block enters as an XOR of address bits below the row stride: offset(ks) = offset(0) ^ 32*ks for K,
  // offset(db) = offset(0) ^ 64*db for V.  A lane keeps the two offsets of step / block 0 (laundered through
  // an empty asm so that they are not recomputed per read); per tile one add forms base + slot (slots are
  // multiples of 4 KB), and a read is that ^ a constant, plus a constant in the instruction's offset field.
  unsigned kb_off0 = (unsigned)(l32 * LF_D * 2 + 16 * lf_k_phys(l32, g));
  asm volatile("" : "+v"(kb_off0));
  unsigned vb_off0;
  {
    const int j16 = lane & 15, dh = (lane >> 4) & 1, row0 = 4 * g + (j16 >> 2);
    const int col = 16 * dh + 4 * (j16 & 3);
    vb_off0 = (unsigned)(row0 * LF_D * 2 + 16 * lf_v_phys(row0, col / 8) + 2 * (col % 8));
    asm volatile("" : "+v"(vb_off0));
  }
  static_assert((LF_BN * LF_D * 2) % 4096 == 0, "slot strides keep the swizzled address bits clear");
  typedef __attribute__((address_space(3))) const lf_u32x4* lf_lds_u32x4_ptr;
  typedef __attribute__((address_space(3))) lf_s16x4* lf_lds_s16x4_ptr;
  // K fragment f = (16-dim step ks, 32-row block kb): rows 32*kb + l32, as lf_read_k_frag; `ka` = LDS address
  // of the tile + kb_off0
  auto k_frag = [&](unsigned ka, int f) {
    const int ks = f / LF_NKB, kb = f % LF_NKB;
    return *(lf_lds_u32x4_ptr)(size_t)((ka ^ (unsigned)(32 * ks)) + (unsigned)(kb * 32 * LF_D * 2));
  };
  // V^T fragment f = (16-key step kk, 32-dim block db), two transposed 8-byte reads, as lf_read_v_frag_tr;
  // `va` = LDS address of the tile + vb_off0
  auto v_frag = [&](unsigned va, int f) {
    const int kk = f / LF_NDB, db = f % LF_NDB;
    lf_elem8 a;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const unsigned src = (va ^ (unsigned)(64 * db)) + (unsigned)((16 * kk + 8 * half) * LF_D * 2);
      lf_s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lf_lds_s16x4_ptr)(size_t)src);
      lf_elem4 te = __builtin_bit_cast(lf_elem4, t);
      a[4 * half + 0] = te[0];
      a[4 * half + 1] = te[1];
      a[4 * half + 2] = te[2];
      a[4 * half + 3] = te[3];
    }
    return a;
  };

  auto run_q_tile = [&](const int qt) {
    const int q0 = qt * LF_BM;
    const int qlast = min(q0 + LF_BM, p.Sq) - 1;
    // ---- block skip: KV tiles [kt_begin, kt_end) hold an unmasked (i, j) for rows q0..qlast
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
#if LF_BIAS
    // tile classes of the bias for this (batch, head, q tile): broadcast dims of the bias collapse
    const int nhh = p.bias_sh ? p.Hq : 1;
    const int cunit = ((p.bias_sb ? b : 0) * nhh + (p.bias_sh ? h : 0)) * nqt + qt;
    const lf_cint* ccls = reinterpret_cast<const lf_cint*>(reinterpret_cast<unsigned long long>(p.part_acc)) +
                          (long long)cunit * nkt;
    {
      // the q tile's range shrinks to its first .. last tile that is not dead (every wave scans for
      // itself, 64 tiles per step: no exchange needed)
      const int* vcls = reinterpret_cast<const int*>(p.part_acc) + (long long)cunit * nkt;
      int lo = kt_end, hi = kt_begin;
      for (int t0 = kt_begin; t0 < kt_end; t0 += 64) {
        const int t = t0 + lane;
        const unsigned long long live = __builtin_amdgcn_ballot_w64(t < kt_end && vcls[min(t, kt_end - 1)] != 0);
        if (live != 0ull) {
          lo = min(lo, t0 + (int)__builtin_ctzll(live));
          hi = t0 + 64 - (int)__builtin_clzll(live);
        }
      }
      kt_begin = min(lo, kt_end);
      kt_end = max(hi, kt_begin);
      kt_begin = __builtin_amdgcn_readfirstlane(kt_begin);
      kt_end = __builtin_amdgcn_readfirstlane(kt_end);
    }
#endif
    if (p.visits != nullptr && tid == 0) {
      for (int kt = kt_begin; kt < kt_end; ++kt)
        p.visits[((long long)bh * nqt + qt) * nkt + kt] = 1;
    }

    const int wq0 = q0 + 32 * (LF_GQAPACK ? wave / LF_GQAPACK : wave);
    const int wqlast = min(wq0 + 31, p.Sq - 1);
    const bool wave_has_rows = wq0 < p.Sq;
    const int my_q = wq0 + l32;

    // ---- prologue: K(begin), K(begin+1), V(begin) resident; first K fragments in flight.
    // The direct loads go out before the Q fetch, so the q tile pays one memory latency
    // instead of two (the memory counter retires in order: the compiler's wait for the Q
    // registers, which counts only the loads it knows, also covers the older direct loads).
    // Paged operands: page offsets of the passes issued during the coming tile (K two
    // tiles ahead, V one tile ahead), fetched a tile before they are needed
    unsigned kpg[LF_NPASS], vpg[LF_NPASS];
    {
      unsigned k0pg[LF_NPASS], k1pg[LF_NPASS], v0pg[LF_NPASS];
#pragma unroll
      for (int ps = 0; ps < LF_NPASS; ++ps) {
        k0pg[ps] = kPagedK ? page_off(0, kt_begin, ps) : 0u;
        k1pg[ps] = kPagedK ? page_off(0, kt_begin + 1, ps) : 0u;
        v0pg[ps] = kPagedV ? page_off(1, kt_begin, ps) : 0u;
        kpg[ps] = kPagedK ? page_off(0, kt_begin + 2, ps) : 0u;
        vpg[ps] = kPagedV ? page_off(1, kt_begin + 1, ps) : 0u;
      }
#pragma unroll
      for (int ps = 0; ps < LF_NPASS; ++ps) {
        dma_k_pass(k_rsq, kt_begin, 0, ps, k0pg[ps]);
        if (kt_begin + 1 < kt_end) dma_k_pass(k_rsq, kt_begin + 1, 1, ps, k1pg[ps]);
        dma_v_pass(v_rsq, kt_begin, 0, ps, v0pg[ps]);
      }
    }
    // Q^T fragments (B operand): lane holds row my_q, d = 16*ks + 8*g .. +7.
    lf_elem8 qf[LF_NKS];
    {
      const lf_elem* qrow = p.q + (long long)b * p.q_sb + (long long)h * p.q_sh +
                            (long long)min(my_q, p.Sq - 1) * p.q_ss;
#pragma unroll
      for (int ks = 0; ks < LF_NKS; ++ks)
        qf[ks] = __builtin_bit_cast(lf_elem8, *reinterpret_cast<const lf_u32x4*>(qrow + 16 * ks + 8 * g));
    }
    // the compiler waits for the Q loads here (a use it can see) and all older vector
    // memory operations are drained, so its bookkeeping is clear before the direct
    // loads of the tile loop, which it does not track, start
#pragma unroll
    for (int ks = 0; ks < LF_NKS; ++ks) asm volatile("" :: "v"(qf[ks]));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    lf_f32x16 o[LF_NDB];
#pragma unroll
    for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] = 0.0f;
    float mc_ref = LF_NEG_INF;   // exponent offset of this query, log2 units (a lagging running max)
    float mc_sub = 0.0f;         // what the exponentials subtract: mc_ref, or 0 while it is still -inf
    float l_run = 0.0f;          // this lane's share of the running sum

    LF_BARRIER_VM0();
    lf_u32x4 kpre[LF_KPF];
#pragma unroll
    for (int f = 0; f < LF_KPF; ++f) kpre[f] = k_frag(k_row_addr(0, 0) + kb_off0, f);

    int ks_cur = 0;   // K slot of tile kt
    for (int kt = kt_begin; kt < kt_end; ++kt) {
      const int rel = kt - kt_begin;
      const int ks_nxt = (ks_cur == LF_KSLOTS - 1) ? 0 : ks_cur + 1;   // slot of K(kt+1)
      const int ks_ld = (ks_nxt == LF_KSLOTS - 1) ? 0 : ks_nxt + 1;    // slot K(kt+2) is loaded into
      const unsigned kbuf = k_row_addr(ks_cur, 0) + kb_off0;       // lane's fragment base in K(kt), K(kt+1), V(kt)
      const unsigned knext = k_row_addr(ks_nxt, 0) + kb_off0;
      const unsigned vbuf = v_row_addr(rel & 1, 0) + vb_off0;
      const int vs_ld = (rel + 1) & 1;                                 // slot V(kt+1) is loaded into
      // direct load number d of this tile: K(kt+2) passes, then V(kt+1) passes.  Tiles past the
      // last one are asked for with an empty range instead of a test per load: a branch between the
      // MFMAs ends the compiler's knowledge of what is in flight
      lf_u32x4 k_cur = k_rsq, v_cur = v_rsq;
      if (kt + 2 >= kt_end) k_cur[2] = 0u;
      if (kt + 1 >= kt_end) v_cur[2] = 0u;
      auto dma_step = [&](int d) {
        if (d < LF_NPASS) dma_k_pass(k_cur, kt + 2, ks_ld, d, kpg[d]);
        else dma_v_pass(v_cur, kt + 1, vs_ld, d - LF_NPASS, vpg[d - LF_NPASS]);
      };
      // page offsets for the next tile's loads (table reads: in flight during this tile)
      unsigned kpg_n[LF_NPASS], vpg_n[LF_NPASS];
#pragma unroll
      for (int ps = 0; ps < LF_NPASS; ++ps) {
        kpg_n[ps] = kPagedK ? page_off(0, kt + 3, ps) : 0u;
        vpg_n[ps] = kPagedV ? page_off(1, kt + 2, ps) : 0u;
      }

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

#if LF_BIAS
      // class 2: the tile's bias values are requested before the S^T products.  Element i of block kb is
      // key j = k0 + 32*kb + 8*(i/4) + 4*g + i%4 of row my_q: four consecutive keys per 8-byte load
      // class 0 inside the range (a dead tile between live ones): staged like any tile, not computed
      const int tile_class = (int)ccls[kt];
      need = need && tile_class != 0;
      const bool biased = need && tile_class == 2;
      lf_u32x2 bias_v[LF_NKB][4];
      if (biased) {
        const lf_elem* brow = p.bias + (long long)b * p.bias_sb + (long long)h * p.bias_sh +
                              (long long)min(my_q, p.Sq - 1) * p.bias_sq;
#pragma unroll
        for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const int j0 = k0 + 32 * kb + 8 * i4 + 4 * g;
            bias_v[kb][i4] = *reinterpret_cast<const lf_u32x2*>(brow + min(j0, p.Sk - 4));
          }
      }
#endif
      if (need) {
        // ---- S^T = K Q^T; the two accumulator chains alternate
        lf_f32x16 s[LF_NKB];
#pragma unroll
        for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[kb][i] = 0.0f;
        lf_u32x4 kf[LF_NFK];
        lf_elem8 vf[LF_NFV];
#pragma unroll
        for (int f = 0; f < LF_KPF; ++f) kf[f] = kpre[f];
#if LF_SETPRIO
        __builtin_amdgcn_s_setprio(2);
#endif
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int f = 0; f < LF_NFK; ++f) {
          if (f + LF_KPF < LF_NFK) kf[f + LF_KPF] = k_frag(kbuf, f + LF_KPF);
          if (f >= LF_NFK - LF_VPF) vf[f - (LF_NFK - LF_VPF)] = v_frag(vbuf, f - (LF_NFK - LF_VPF));
          if (f % (LF_NFK / (2 * LF_NPASS)) == 1) dma_step(f / (LF_NFK / (2 * LF_NPASS)));
          s[f % LF_NKB] = lf_mfma32(__builtin_bit_cast(lf_elem8, kf[f]), qf[f / LF_NKB], s[f % LF_NKB]);
          __builtin_amdgcn_sched_barrier(0);
        }
#if LF_SETPRIO
        __builtin_amdgcn_s_setprio(0);
#endif

        // ---- score modifications and mask; element i of block kb is kv index
        // j = k0 + 32*kb + 8*(i/4) + 4*g + i%4, query my_q.
#if LF_CAPPOLY
        // largest |raw score| of the wave's tile: decides between the polynomial and the exact form
        float amax = 0.0f;
#pragma unroll
        for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(s[kb][i]));
        const bool cap_fused = __builtin_amdgcn_ballot_w64(!(amax <= cap_smax)) == 0ull && full;
        // coefficients of the exponent's polynomial for this tile: the cap's, or the identity for a tile that is
        // transformed in place (tiny positive instead of 0: a masked score, -inf, then stays -inf instead of NaN)
        float kA0 = capA0, kA1 = capA1;
#if LF_CAP_TERMS >= 2
        float kA2 = capA2;
#endif
        if (!cap_fused) {
          if (__builtin_amdgcn_ballot_w64(!(amax <= cap_smax2)) == 0ull) {
#pragma unroll
            for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
              for (int i = 0; i < 16; ++i) {
                const float u = s[kb][i] * s[kb][i];
                s[kb][i] *= __builtin_fmaf(u, __builtin_fmaf(u, capP2, capP1), capA0);
              }
          } else {
#pragma unroll
            for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
              for (int i = 0; i < 16; ++i)
                s[kb][i] = __builtin_fmaf(__builtin_amdgcn_rcpf(-1.0f - lf_exp2(s[kb][i] * sc_exp)), 2.0f * cap_l2, cap_l2);
          }
          kA0 = 1.0f;
          kA1 = 1e-30f;
#if LF_CAP_TERMS >= 2
          kA2 = 1e-30f;
#endif
        }
        // c*log2e*tanh of a raw score (or the identity), as a factor: score * cap_t(score^2)
        auto cap_t = [&](float u) {
#if LF_CAP_TERMS >= 2
          return __builtin_fmaf(u, __builtin_fmaf(u, kA2, kA1), kA0);
#else
          return __builtin_fmaf(u, kA1, kA0);
#endif
        };
#elif LF_SOFTCAP
#pragma unroll
        for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[kb][i] = __builtin_amdgcn_rcpf(-1.0f - lf_exp2(s[kb][i] * sc_exp));   // -r
#endif
#if LF_BIAS
        if (biased) {
          // x = scale * s + bias: the scores stay in units of 1 / scale, so the bias is divided by it; capped
          // scores are held as -r with c * tanh = c - 2 c r: there the unit is 2 c
#if LF_SOFTCAP
          const float inv_scale = 0.5f / p.softcap;
#else
          const float inv_scale = 1.0f / p.scale;
#endif
#pragma unroll
          for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
              const int j0 = k0 + 32 * kb + 8 * i4 + 4 * g;
              const lf_elem4 bv = __builtin_bit_cast(lf_elem4, bias_v[kb][i4]);
              // a tile that ends past Sk was read from Sk - 4: keys beyond Sk are masked below anyway
              const int sh = j0 - min(j0, p.Sk - 4);
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float bval = lf_bias_value(sh == 0 ? bv[e] : bv[min(e + sh, 3)]);
                s[kb][4 * i4 + e] += bval * inv_scale;
              }
            }
        }
#endif
        if (!full) {
          // key j = k0 + 4*g + c with the compile-time c = 32*kb + 8*(i/4) + i%4: the bound j < Sk and the
          // causal j <= my_q fold into one per-lane limit, so an element costs one compare against an
          // inline constant (the window, i - j < w, a second one)
          int hi = p.Sk - 1 - k0 - 4 * g;
#if LF_MASK >= 1
          hi = min(hi, my_q - k0 - 4 * g);
#endif
#if LF_MASK == 2
          const int lo = my_q - k0 - 4 * g - p.window;       // c > lo
#endif
#pragma unroll
          for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int c = 32 * kb + 8 * (i / 4) + (i % 4);
#if LF_MASK == 2
              const bool ok = c <= hi && c > lo;
#else
              const bool ok = c <= hi;
#endif
              s[kb][i] = ok ? s[kb][i] : LF_NEG_INF;
            }
        }

        // ---- online softmax with a lagging offset (see lf_attn_prefill.hip)
        float mx = LF_NEG_INF;
#pragma unroll
        for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kb][i]);
        mx = lf_max_halves(mx);
#if LF_CAPPOLY
        const float mxc = mx * cap_t(mx * mx);
#else
        const float mxc = mx * cexp;
#endif
        if (__builtin_amdgcn_ballot_w64(mxc > mc_ref + (float)LF_LAZY_LOG2) != 0ull) {
          const float mc_new = fmaxf(mc_ref, mxc);
          const float r = (mc_new == LF_NEG_INF) ? 1.0f : lf_exp2(mc_ref - mc_new);
          // no row of the wave has seen a key yet (the first tile of a q tile): O and l are still zero
          const bool fresh = __builtin_amdgcn_ballot_w64(mc_ref != LF_NEG_INF) == 0ull;
          mc_ref = mc_new;
          mc_sub = (mc_new == LF_NEG_INF) ? 0.0f : mc_new;
          if (!fresh) {
            l_run *= r;
#pragma unroll
            for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
              for (int i = 0; i < 16; ++i) o[db][i] *= r;
          }
        }
        float rs = 0.0f;
        lf_elem8 pf[LF_NKK];
        // probabilities number [e0, e1) of the tile in the order the second product consumes them:
        // e = 16 * (key block) + (accumulator element), B operand e / 8
        auto exp_range = [&](int e0, int e1) {
#pragma unroll
          for (int e = e0; e < e1; ++e) {
#if LF_CAPPOLY
            const float sv = s[e / 16][e % 16];
            const float ex = lf_exp2(__builtin_fmaf(sv, cap_t(sv * sv), -mc_sub));
#else
            const float ex = lf_exp2(s[e / 16][e % 16] * cexp - mc_sub);
#endif
            rs += ex;
            pf[e / 8][e % 8] = lf_from_float(ex);
          }
        };
#if LF_SPLIT_EXP
        // the exponentials of the tile's second half go between the MFMAs that consume the first:
        // the wave keeps the matrix pipe busy during half of its own softmax
        exp_range(0, 8 * LF_NKB);
#else
        exp_range(0, 16 * LF_NKB);
#endif

        // ---- O^T += V^T P^T; the last steps also read the first fragments of K(kt+1)
#if LF_SETPRIO
        __builtin_amdgcn_s_setprio(2);
#endif
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int f = 0; f < LF_NFV; ++f) {
          if (f + LF_VPF < LF_NFV) vf[f + LF_VPF] = v_frag(vbuf, f + LF_VPF);
          if (f >= LF_NFV - LF_KPF) kpre[f - (LF_NFV - LF_KPF)] = k_frag(knext, f - (LF_NFV - LF_KPF));
          o[f % LF_NDB] = lf_mfma32(vf[f], pf[f / LF_NDB], o[f % LF_NDB]);
#if LF_SPLIT_EXP
          if (f < LF_NFV / 2) exp_range(8 * LF_NKB + f * (16 * LF_NKB) / LF_NFV, 8 * LF_NKB + (f + 1) * (16 * LF_NKB) / LF_NFV);
#endif
          __builtin_amdgcn_sched_barrier(0);
        }
        l_run += rs;
#if LF_SETPRIO
        __builtin_amdgcn_s_setprio(0);
#endif
      } else {
        // this wave's rows see nothing of tile kt: it only stages and reads ahead
#pragma unroll
        for (int d = 0; d < 2 * LF_NPASS; ++d) dma_step(d);
#pragma unroll
        for (int f = 0; f < LF_KPF; ++f) kpre[f] = k_frag(knext, f);
      }
      LF_BARRIER_VM0();
      ks_cur = ks_nxt;
#pragma unroll
      for (int ps = 0; ps < LF_NPASS; ++ps) {
        kpg[ps] = kpg_n[ps];
        vpg[ps] = vpg_n[ps];
      }
    }

    // ---- epilogue: O[q][d] = O^T[d][q] / l.  Element i of block db is
    // d = 32*db + 8*(i/4) + 4*g + i%4.
    const float l_tot = l_run + lf_swap32(l_run);
    // optional: the row's log-sum-exp of the scaled, masked scores in log2 units (what a
    // backward pass recomputes the probabilities from); -inf for a row that saw no key
    if (p.part_ml != nullptr && g == 0 && my_q < p.Sq)
#if LF_SOFTCAP && !LF_CAPPOLY
      // the kernel's scores are the capped ones minus the cap: the cap comes back in here
      p.part_ml[((long long)b * p.Hq + h) * p.Sq + my_q] = mc_ref + __builtin_log2f(l_tot) + p.softcap * LF_LOG2E;
#else
      p.part_ml[((long long)b * p.Hq + h) * p.Sq + my_q] = mc_ref + __builtin_log2f(l_tot);
#endif
    {
      // Lane (q, g) holds, per block db, four 4-value chunks d = 32*db + 8*i4 + 4*g + 0..3.
      // One v_permlane32_swap per register pair trades chunks with the lane that holds
      // the other half of the same row, so that each lane owns 8 consecutive d's and
      // writes them with one 16-byte store (32 contiguous bytes per row and instruction).
#if LF_SAFE
      const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;      // a row that saw no key gives zeros
#else
      const float inv = 1.0f / l_tot;
#endif
      lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)h * p.o_sh +
                      (long long)min(my_q, p.Sq - 1) * p.o_ss;
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db) {
        unsigned ch[4][2];
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          lf_elem4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = lf_from_float(o[db][4 * i4 + e] * inv);
          const lf_u32x2 wu = __builtin_bit_cast(lf_u32x2, w);
          ch[i4][0] = wu[0];
          ch[i4][1] = wu[1];
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          auto r0 = __builtin_amdgcn_permlane32_swap(ch[2 * j][0], ch[2 * j + 1][0], false, false);
          auto r1 = __builtin_amdgcn_permlane32_swap(ch[2 * j][1], ch[2 * j + 1][1], false, false);
          const lf_u32x4 out = {r0[0], r1[0], r0[1], r1[1]};
          if (my_q < p.Sq) *reinterpret_cast<lf_u32x4*>(orow + 32 * db + 16 * j + 8 * g) = out;
        }
      }
    }
  };

  run_q_tile(slot_qt);
}
