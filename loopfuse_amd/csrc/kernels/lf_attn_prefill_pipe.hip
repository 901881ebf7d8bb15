// lf_attn_prefill_pipe.hip — software-pipelined fused attention forward for
// gfx950 (prefill shapes), one wave per SIMD.
//
// Workgroup = 4 waves x 64 query rows (two 32-row halves per wave), KV tiles of
// 64 rows double-buffered in XOR-swizzled LDS (K ring and V ring, 2 slots each).
// As in lf_attn_prefill.hip the wave works on the transposed problem
//     S^T = K Q^T ,  O^T += V^T P^T        (v_mfma_f32_32x32x16)
// so P stays in registers and every per-query quantity is a per-lane scalar.
// Two things differ:
//   * each K / V fragment read from LDS feeds TWO MFMAs (one per 32-row half),
//     halving LDS traffic per flop -- at one fragment per MFMA the 128 B/clk
//     LDS port saturates at the same time as the matrix pipe;
//   * the KV loop is skewed so that the matrix pipe and the vector ALU of the one
//     resident wave overlap: step s issues
//         QK^T of tile s+1   |  softmax of tile s, half 0
//         PV   of tile s-1   |  softmax of tile s, half 1
//     i.e. both MFMA batches are independent of the VALU work issued beside them.
//     (The loop nest is still the reference's fused nest -- loopfuse/compiler/
//     passes/factor_acc.py:23-109 -- with its steps re-timed.)
// The softmax offset lags the running max by up to 2^LF_LAZY_LOG2, so O is
// rescaled (after the PV of the step) only when a wave-uniform test fires.
// Tile bounds (block skip) are those of loopfuse/compiler/passes/
// skip_loop_iterations.py:343-376 in closed form.

#ifndef LF_LAZY_LOG2
#define LF_LAZY_LOG2 8
#endif

#define LF_QH 2                              /* 32-row halves per wave         */
#define LF_NW 4
#define LF_NT (LF_NW * 64)
#define LF_BM (32 * LF_QH * LF_NW)           /* 256 query rows per workgroup   */
#ifndef LF_BN
#define LF_BN 32
#endif
#define LF_D LF_HEAD_DIM
#define LF_CPR (LF_D / 8)
#define LF_RPS (256 / (LF_D * 2))
#define LF_NPASS (LF_BN * LF_CPR / LF_NT)
#define LF_NKB (LF_BN / 32)
#define LF_NKS (LF_D / 16)
#define LF_NDB (LF_D / 32)
#define LF_NKK (LF_BN / 16)

__device__ __forceinline__ int lf_k_phys(int row, int ch) {
  return ch ^ ((row / LF_RPS) & (LF_CPR - 1));
}
__device__ __forceinline__ int lf_v_phys(int row, int ch) {
  return ch ^ (4 * ((row / LF_RPS) & (LF_CPR / 4 - 1)));
}

struct LfScores { lf_f32x16 v[LF_QH][LF_NKB]; };   // S^T of one KV tile, both halves
struct LfProbs  { lf_elem8 v[LF_QH][LF_NKK]; };    // P^T of one KV tile as B operands

extern "C" __global__ void __launch_bounds__(LF_NT, 1) lf_attn_prefill_pipe(const LfAttnParams p) {
  __shared__ __attribute__((aligned(16))) lf_elem lds_k[2][LF_BN * LF_D];
  __shared__ __attribute__((aligned(16))) lf_elem lds_v[2][LF_BN * LF_D];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // ---- workgroup -> (batch*head, q tile); all q tiles of a (batch, head) share an
  // XCD (ids with equal id%8), heaviest q tile first
  const int nqt = (p.Sq + LF_BM - 1) / LF_BM;
  const int nbh = p.B * p.Hq;
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  const int grp = slot / (4 * nqt);
  const int in_grp = slot % (4 * nqt);
  const int bh = (grp * 4 + (in_grp & 3)) * 8 + xcd;
  if (bh >= nbh) return;
  const int qt = nqt - 1 - (in_grp >> 2);
  const int b = bh / p.Hq;
  const int h = bh % p.Hq;
  const int hkv = h / (p.Hq / p.Hkv);
  const int q0 = qt * LF_BM;
  const int qlast = min(q0 + LF_BM, p.Sq) - 1;
  const int nkt = (p.Sk + LF_BN - 1) / LF_BN;

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

  const int wq0 = q0 + 32 * LF_QH * wave;
  const int wqlast = min(wq0 + 32 * LF_QH - 1, p.Sq - 1);
  const bool wave_has_rows = wq0 < p.Sq;

  // Q^T fragments: half hh, lane holds row wq0 + 32*hh + l32, d = 16*ks + 8*g .. +7
  lf_elem8 qf[LF_QH][LF_NKS];
#pragma unroll
  for (int hh = 0; hh < LF_QH; ++hh) {
    const int qi = min(wq0 + 32 * hh + l32, p.Sq - 1);     // rows past Sq duplicate the last one
    const lf_elem* qrow = p.q + (long long)b * p.q_sb + (long long)h * p.q_sh + (long long)qi * p.q_ss;
#pragma unroll
    for (int ks = 0; ks < LF_NKS; ++ks)
      qf[hh][ks] = __builtin_bit_cast(lf_elem8, *reinterpret_cast<const lf_u32x4*>(qrow + 16 * ks + 8 * g));
  }

#if LF_SOFTCAP
  const float sc_in = p.scale / p.softcap;
  const float cexp = LF_LOG2E;
#else
  const float cexp = p.scale * LF_LOG2E;
#endif

  lf_f32x16 o[LF_QH][LF_NDB];
#pragma unroll
  for (int hh = 0; hh < LF_QH; ++hh)
#pragma unroll
    for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[hh][db][i] = 0.0f;
  float mc_ref[LF_QH], l_run[LF_QH];
#pragma unroll
  for (int hh = 0; hh < LF_QH; ++hh) {
    mc_ref[hh] = LF_NEG_INF;
    l_run[hh] = 0.0f;
  }

  // ---- staging (global -> registers -> LDS), one 16-byte chunk per thread and pass
  lf_u32x4 kst[LF_NPASS], vst[LF_NPASS];
  constexpr int kRowsPerPass = LF_NT / LF_CPR;
  const int srow = tid / LF_CPR;
  const int sch = tid % LF_CPR;
  const lf_elem* k_uni = p.k + (long long)b * p.k_sb + (long long)hkv * p.k_sh;
  const lf_elem* v_uni = p.v + (long long)b * p.v_sb + (long long)hkv * p.v_sh;
  const unsigned k_toff = (unsigned)(srow * p.k_ss) + 8u * sch;
  const unsigned v_toff = (unsigned)(srow * p.v_ss) + 8u * sch;

  auto load_k = [&](int kt) {
    const bool tail = (kt + 1) * LF_BN > p.Sk;
#pragma unroll
    for (int ps = 0; ps < LF_NPASS; ++ps) {
      const int r0 = kt * LF_BN + kRowsPerPass * ps;
      if ((LF_PAGED & 1) || tail) {
        const int tok = min(r0 + srow, p.Sk - 1);      // masked rows: any finite data
        kst[ps] = *reinterpret_cast<const lf_u32x4*>(lf_kv_row(p, 0, b, hkv, tok) + 8 * sch);
      } else {
        kst[ps] = *reinterpret_cast<const lf_u32x4*>(k_uni + (long long)r0 * p.k_ss + k_toff);
      }
    }
  };
  auto load_v = [&](int kt) {
    const bool tail = (kt + 1) * LF_BN > p.Sk;
#pragma unroll
    for (int ps = 0; ps < LF_NPASS; ++ps) {
      const int r0 = kt * LF_BN + kRowsPerPass * ps;
      if ((LF_PAGED & 2) || tail) {
        const int tok = min(r0 + srow, p.Sk - 1);
        vst[ps] = *reinterpret_cast<const lf_u32x4*>(lf_kv_row(p, 1, b, hkv, tok) + 8 * sch);
      } else {
        vst[ps] = *reinterpret_cast<const lf_u32x4*>(v_uni + (long long)r0 * p.v_ss + v_toff);
      }
    }
  };
  auto store_k = [&](int kt) {
#pragma unroll
    for (int ps = 0; ps < LF_NPASS; ++ps) {
      const int row = srow + kRowsPerPass * ps;
      *reinterpret_cast<lf_u32x4*>(&lds_k[kt & 1][row * LF_D + 8 * lf_k_phys(row, sch)]) = kst[ps];
    }
  };
  auto store_v = [&](int kt) {
#pragma unroll
    for (int ps = 0; ps < LF_NPASS; ++ps) {
      const int row = srow + kRowsPerPass * ps;
      *reinterpret_cast<lf_u32x4*>(&lds_v[kt & 1][row * LF_D + 8 * lf_v_phys(row, sch)]) = vst[ps];
    }
  };

  // ---- per-tile predicates of this wave
  auto tile_need = [&](int kt) {
    const int k0 = kt * LF_BN;
    bool need = wave_has_rows && kt >= kt_begin && kt < kt_end;
#if LF_MASK >= 1
    need = need && (k0 <= wqlast);
#endif
#if LF_MASK == 2
    need = need && (min(k0 + LF_BN, p.Sk) - 1 >= wq0 - p.window + 1);
#endif
    return need;
  };
  auto tile_full = [&](int kt) {
    const int k0 = kt * LF_BN;
    bool full = (k0 + LF_BN <= p.Sk);
#if LF_MASK >= 1
    full = full && (k0 + LF_BN - 1 <= wq0);
#endif
#if LF_MASK == 2
    full = full && (wq0 + 32 * LF_QH - 1 - k0 < p.window);
#endif
    return full;
  };

  // ---- the three pipeline stages
  auto qk = [&](int kt, LfScores& S) {
    const lf_elem* kbuf = lds_k[kt & 1];
#pragma unroll
    for (int hh = 0; hh < LF_QH; ++hh)
#pragma unroll
      for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) S.v[hh][kb][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < LF_NKS; ++ks)
#pragma unroll
      for (int kb = 0; kb < LF_NKB; ++kb) {
        const int row = 32 * kb + l32;
        const lf_elem8 a = __builtin_bit_cast(
            lf_elem8, *reinterpret_cast<const lf_u32x4*>(&kbuf[row * LF_D + 8 * lf_k_phys(row, 2 * ks + g)]));
#pragma unroll
        for (int hh = 0; hh < LF_QH; ++hh) S.v[hh][kb] = lf_mfma32(a, qf[hh][ks], S.v[hh][kb]);
      }
  };

  // softmax of half hh of tile kt: S -> P, updates (mc_ref, l_run); returns the
  // factor O[hh] has to be multiplied with once the PV of tile kt-1 is in
  auto softmax_half = [&](int kt, int hh, bool masked, LfScores& S, LfProbs& P) -> float {
    const int my_q = wq0 + 32 * hh + l32;
    const int k0 = kt * LF_BN;
#if LF_SOFTCAP
#pragma unroll
    for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) S.v[hh][kb][i] = p.softcap * lf_tanh(S.v[hh][kb][i] * sc_in);
#endif
    if (masked) {
#pragma unroll
      for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int j = k0 + 32 * kb + 8 * (i / 4) + 4 * g + (i % 4);
          bool ok = j < p.Sk;
#if LF_MASK >= 1
          ok = ok && (j <= my_q);
#endif
#if LF_MASK == 2
          ok = ok && (my_q - j < p.window);
#endif
          S.v[hh][kb][i] = ok ? S.v[hh][kb][i] : LF_NEG_INF;
        }
    }
    float mx = LF_NEG_INF;
#pragma unroll
    for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, S.v[hh][kb][i]);
    mx = fmaxf(mx, lf_swap32(mx));
    const float mxc = mx * cexp;
    const float mc_old = mc_ref[hh];
    const float mc_new = (mxc > mc_old + (float)LF_LAZY_LOG2) ? fmaxf(mc_old, mxc) : mc_old;
    const float r = (mc_new == mc_old) ? 1.0f : lf_exp2(mc_old - mc_new);
    mc_ref[hh] = mc_new;
    const float mc_sub = (mc_new == LF_NEG_INF) ? 0.0f : mc_new;
    float rs = 0.0f;
#pragma unroll
    for (int kb = 0; kb < LF_NKB; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float e = lf_exp2(S.v[hh][kb][i] * cexp - mc_sub);
        rs += e;
        P.v[hh][2 * kb + i / 8][i % 8] = lf_from_float(e);
      }
    l_run[hh] = l_run[hh] * r + rs;
    return r;
  };

  auto pv = [&](int kt, const LfProbs& P) {
    const lf_elem* vbuf = lds_v[kt & 1];
    const int j16 = lane & 15;
    const int dh = (lane >> 4) & 1;
#pragma unroll
    for (int kk = 0; kk < LF_NKK; ++kk)
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db) {
        // V^T fragment (A operand, row = d): two transposed 8-byte reads, see
        // lf_attn_prefill.hip for the lane/row assignment
        lf_elem8 a;
        const int col = 32 * db + 16 * dh + 4 * (j16 & 3);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int row = 16 * kk + 8 * half + 4 * g + (j16 >> 2);
          const lf_elem* src = &vbuf[row * LF_D + 8 * lf_v_phys(row, col / 8) + (col % 8)];
          lf_s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(src));
          lf_elem4 te = __builtin_bit_cast(lf_elem4, t);
          a[4 * half + 0] = te[0];
          a[4 * half + 1] = te[1];
          a[4 * half + 2] = te[2];
          a[4 * half + 3] = te[3];
        }
#pragma unroll
        for (int hh = 0; hh < LF_QH; ++hh) o[hh][db] = lf_mfma32(a, P.v[hh][kk], o[hh][db]);
      }
  };

  auto rescale = [&](const float (&r)[LF_QH]) {
    bool any = false;
#pragma unroll
    for (int hh = 0; hh < LF_QH; ++hh) any = any || (r[hh] != 1.0f);
    if (__builtin_amdgcn_ballot_w64(any) != 0ull) {
#pragma unroll
      for (int hh = 0; hh < LF_QH; ++hh)
#pragma unroll
        for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[hh][db][i] *= r[hh];
    }
  };

  // one skewed step: QK(s+1) -> Snext, softmax(s): Scur -> Pnew, PV(s-1) with Pold
  auto step = [&](int s, LfScores& Scur, LfScores& Snext, const LfProbs& Pold, LfProbs& Pnew) {
    if (s + 2 < kt_end) load_k(s + 2);
    const bool v_now = s >= kt_begin && s < kt_end;
    if (v_now) load_v(s);

    const bool do_qk = tile_need(s + 1);
    const bool do_sm = tile_need(s);
    const bool do_pv = tile_need(s - 1);
    float r[LF_QH];
#pragma unroll
    for (int hh = 0; hh < LF_QH; ++hh) r[hh] = 1.0f;

    if (do_qk && do_sm && do_pv && tile_full(s)) {
      // steady state: one straight-line block, MFMA batches beside independent VALU work
      qk(s + 1, Snext);
      r[0] = softmax_half(s, 0, false, Scur, Pnew);
      pv(s - 1, Pold);
      r[1] = softmax_half(s, 1, false, Scur, Pnew);
    } else {
      if (do_qk) qk(s + 1, Snext);
      if (do_sm) {
        const bool masked = !tile_full(s);
#pragma unroll
        for (int hh = 0; hh < LF_QH; ++hh) r[hh] = softmax_half(s, hh, masked, Scur, Pnew);
      }
      if (do_pv) pv(s - 1, Pold);
    }
    rescale(r);

    if (s + 2 < kt_end) store_k(s + 2);
    if (v_now) store_v(s);
    __syncthreads();
  };

  // ---- prologue: K of the first tile
  load_k(kt_begin);
  store_k(kt_begin);
  __syncthreads();

  LfScores SA, SB;
  LfProbs PA, PB;
  // steps kt_begin-1 .. kt_end, two per trip so the register roles alternate statically
  for (int s = kt_begin - 1; s <= kt_end; s += 2) {
    step(s, SA, SB, PA, PB);
    if (s + 1 <= kt_end) step(s + 1, SB, SA, PB, PA);
  }

  // ---- epilogue: O[q][d] = O^T[d][q] / l
#pragma unroll
  for (int hh = 0; hh < LF_QH; ++hh) {
    const int my_q = wq0 + 32 * hh + l32;
    const float l_tot = l_run[hh] + lf_swap32(l_run[hh]);
    if (my_q < p.Sq) {
      const float inv = 1.0f / l_tot;
      lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)h * p.o_sh + (long long)my_q * p.o_ss;
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db)
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          lf_elem4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = lf_from_float(o[hh][db][4 * i4 + e] * inv);
          *reinterpret_cast<lf_elem4*>(orow + 32 * db + 8 * i4 + 4 * g) = w;
        }
    }
  }
}
