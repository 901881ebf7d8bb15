// lf_attn_decode.hip — split-K decode attention for gfx950 (few query rows per
// (batch, kv head), long KV): a pure HBM-streaming kernel.
//
// A "unit" is one (batch, kv head, row chunk): LF_ROWS (1, 2 or 4) query rows
// that share every K/V fetch (GQA group rows, reference benchmark.py:439-443).
// grid = (units, nsplit); a workgroup of LF_DW waves owns tokens
// [z*split_len, (z+1)*split_len) of its unit and deals them to its waves in
// 16-token steps.  Per step a lane (t = lane%16, g = lane/16) loads, straight
// from global memory into registers and 16 bytes at a time, the pieces
// d = 32*j + 8*g .. +7 (j < D/32) of K[token t] and V[token t].  Those registers
// ARE the B operand of v_mfma_f32_16x16x32 (column = token, k = d), so
//     S[row, t] = sum_d Q[row, d] K[t, d]
// costs D/32 MFMAs with Q (rows replicated to fill 16) as the A operand, and
// every lane ends up holding the scores of all LF_ROWS rows for ITS token.  Each
// lane keeps a private online-softmax state (m, l, acc[row][its 32 d's]) for
// the tokens it has seen; PV is plain FMAs on the V registers.  No LDS, no
// barrier and no cross-lane traffic inside the loop.  At the end the 16 token
// lanes of each wave and the waves of the workgroup are merged through LDS
// with the usual (max, sum, acc) log-sum-exp combine; with nsplit > 1 the
// workgroup writes its partial to scratch and lf_attn_decode_combine merges.
//
// The page-table gather (LF_PAGED) is fused into the row address: page ids for
// step s+2 are fetched while K/V of step s+1 are in flight and step s is
// being consumed (reference: loopfuse/codegen.py:738-872).

#ifndef LF_ROWS
#define LF_ROWS 1
#endif
#ifndef LF_DW
#define LF_DW 4              /* waves per workgroup */
#endif
#define LF_DT (LF_DW * 64)
#define LF_D LF_HEAD_DIM
#define LF_NJ (LF_D / 32)    /* 16-byte pieces of a row held by one lane */

struct LfDecStep {
  lf_u32x4 k[LF_NJ];
  lf_u32x4 v[LF_NJ];
};

extern "C" __global__ void __launch_bounds__(LF_DT, 2) lf_attn_decode(const LfAttnParams p) {
  // merge buffer: [LF_DW*16 (wave, token lane)][LF_D] floats for one row at a time
  __shared__ float red[LF_DW * 16 * LF_D];
  __shared__ float red_m[LF_DW][LF_ROWS];
  __shared__ float red_l[LF_DW][LF_ROWS];
  __shared__ float part_sum[LF_DT / LF_D][LF_D];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int t = lane & 15;
  const int g = lane >> 4;

  const int unit = blockIdx.x;
  const int z = blockIdx.y;
  const int chunks = (p.rows + LF_ROWS - 1) / LF_ROWS;   // row chunks per (b, kv head)
  const int rc = unit % chunks;
  const int bh = unit / chunks;
  const int hkv = bh % p.Hkv;
  const int b = bh / p.Hkv;
  const int row0 = rc * LF_ROWS;                           // first query row of this unit

  const int tok_begin = z * p.split_len;
  const int tok_end = min(tok_begin + p.split_len, p.Sk);
  const int nsteps = (max(tok_end - tok_begin, 0) + 15) / 16;

  // ---- A operand: Q rows replicated, lane (m = lane%16, g) holds
  // Q[row0 + m % LF_ROWS][32*j + 8*g .. +7].  Query row r of the unit is the
  // tensor row (head = hkv*rows + r) when Sq == 1, i.e. Q viewed [B, Hkv, rows, D].
  lf_elem8 qa[LF_NJ];
  {
    int r = row0 + (t % LF_ROWS);
    if (r >= p.rows) r = p.rows - 1;
    const lf_elem* qrow = p.q + (long long)b * p.q_sb + (long long)hkv * p.q_sh + (long long)r * p.q_ss;
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j)
      qa[j] = __builtin_bit_cast(lf_elem8, *reinterpret_cast<const lf_u32x4*>(qrow + 32 * j + 8 * g));
  }

#if LF_SOFTCAP
  const float sc_in = p.scale / p.softcap;
  const float cexp = LF_LOG2E;
#else
  const float cexp = p.scale * LF_LOG2E;
#endif

  float m_run[LF_ROWS], l_run[LF_ROWS];
  float acc[LF_ROWS][LF_NJ][8];
#pragma unroll
  for (int r = 0; r < LF_ROWS; ++r) {
    m_run[r] = LF_NEG_INF;
    l_run[r] = 0.0f;
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[r][j][e] = 0.0f;
  }

  // ---- token stream of this wave: steps wave, wave + LF_DW, ...
  auto step_tok = [&](int s) { return tok_begin + 16 * s + t; };
  auto row_ptrs = [&](int s, const lf_elem*& kp, const lf_elem*& vp) {
    int tok = min(step_tok(s), p.Sk - 1);      // clamp: masked later, never out of bounds
    kp = lf_kv_row(p, 0, b, hkv, tok) + 8 * g;
    vp = lf_kv_row(p, 1, b, hkv, tok) + 8 * g;
  };
  auto issue = [&](LfDecStep& st, const lf_elem* kp, const lf_elem* vp) {
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) st.k[j] = *reinterpret_cast<const lf_u32x4*>(kp + 32 * j);
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) st.v[j] = *reinterpret_cast<const lf_u32x4*>(vp + 32 * j);
  };
  auto consume = [&](const LfDecStep& st, int s) {
    lf_f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) sc = lf_mfma16(qa[j], __builtin_bit_cast(lf_elem8, st.k[j]), sc);
    const bool valid = step_tok(s) < tok_end;
    float vf[LF_NJ][8];
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) {
      lf_elem8 ve = __builtin_bit_cast(lf_elem8, st.v[j]);
#pragma unroll
      for (int e = 0; e < 8; ++e) vf[j][e] = lf_to_float(ve[e]);
    }
#pragma unroll
    for (int r = 0; r < LF_ROWS; ++r) {
      float x = sc[r];                         // C row 4*g + r holds query row r (replicated)
#if LF_SOFTCAP
      x = p.softcap * lf_tanh(x * sc_in);
#endif
      x = valid ? x : LF_NEG_INF;
      const float m_new = fmaxf(m_run[r], x);
      const float m_sub = (m_new == LF_NEG_INF) ? 0.0f : m_new;
      const float mc = m_sub * cexp;
      const float resc = lf_exp2(m_run[r] * cexp - mc);
      const float pe = lf_exp2(x * cexp - mc);
      m_run[r] = m_new;
      l_run[r] = l_run[r] * resc + pe;
#pragma unroll
      for (int j = 0; j < LF_NJ; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][j][e] = acc[r][j][e] * resc + pe * vf[j][e];
    }
  };

  {
    LfDecStep st0, st1;
    const lf_elem *kp, *vp;
    int s = wave;
    if (s < nsteps) {
      row_ptrs(s, kp, vp);
      issue(st0, kp, vp);
    }
    // two steps per trip so both register stages have static names
    for (; s < nsteps; s += 2 * LF_DW) {
      const int s1 = s + LF_DW;
      const int s2 = s + 2 * LF_DW;
      if (s1 < nsteps) {
        row_ptrs(s1, kp, vp);
        issue(st1, kp, vp);
      }
      consume(st0, s);
      if (s2 < nsteps) {
        row_ptrs(s2, kp, vp);
        issue(st0, kp, vp);
      }
      if (s1 < nsteps) consume(st1, s1);
    }
  }

  // ---- merge the 16 token lanes x LF_DW waves.  (m, l) do not depend on g.
  float m_wg[LF_ROWS], l_wg[LF_ROWS];
#pragma unroll
  for (int r = 0; r < LF_ROWS; ++r) {
    float mw = m_run[r];
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off, 64));
    if (lane == 0) red_m[wave][r] = mw;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < LF_ROWS; ++r) {
    float mw = red_m[0][r];
#pragma unroll
    for (int w = 1; w < LF_DW; ++w) mw = fmaxf(mw, red_m[w][r]);
    m_wg[r] = mw;
    const float m_sub = (mw == LF_NEG_INF) ? 0.0f : mw;
    const float f = lf_exp2(m_run[r] * cexp - m_sub * cexp);   // 0 for lanes that saw nothing
    float lw = l_run[r] * f;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) lw += __shfl_xor(lw, off, 64);
    if (lane == 0) red_l[wave][r] = lw;
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[r][j][e] *= f;
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < LF_ROWS; ++r) {
    float lw = red_l[0][r];
#pragma unroll
    for (int w = 1; w < LF_DW; ++w) lw += red_l[w][r];
    l_wg[r] = lw;
  }

  const int dcol = tid % LF_D;          // column this thread sums in the merge
  const int part = tid / LF_D;          // which slice of the (wave, lane) rows
  constexpr int kParts = LF_DT / LF_D;  // 2 for D = 128 with 256 threads
  constexpr int kRowsPerPart = LF_DW * 16 / kParts;
#pragma unroll
  for (int r = 0; r < LF_ROWS; ++r) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) {
      float* dst = &red[(wave * 16 + t) * LF_D + 32 * j + 8 * g];
      *reinterpret_cast<lf_f32x4*>(dst) = lf_f32x4{acc[r][j][0], acc[r][j][1], acc[r][j][2], acc[r][j][3]};
      *reinterpret_cast<lf_f32x4*>(dst + 4) = lf_f32x4{acc[r][j][4], acc[r][j][5], acc[r][j][6], acc[r][j][7]};
    }
    __syncthreads();
    float sum = 0.0f;
#pragma unroll 8
    for (int i = 0; i < kRowsPerPart; ++i) sum += red[(part * kRowsPerPart + i) * LF_D + dcol];
    if (kParts > 1) {
      part_sum[part][dcol] = sum;
      __syncthreads();
      if (part == 0) {
#pragma unroll
        for (int q = 1; q < kParts; ++q) sum += part_sum[q][dcol];
      }
    }
    const int qr = row0 + r;
    if (part == 0 && qr < p.rows) {
      if (p.nsplit == 1) {
        lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)hkv * p.o_sh + (long long)qr * p.o_ss;
        orow[dcol] = lf_from_float(sum / l_wg[r]);
      } else {
        const long long slot = ((long long)bh * p.rows + qr) * p.nsplit + z;
        p.part_acc[slot * LF_D + dcol] = sum;
        if (dcol == 0) {
          p.part_ml[slot * 2 + 0] = m_wg[r] * cexp;   // in exponent units (log2 domain)
          p.part_ml[slot * 2 + 1] = l_wg[r];
        }
      }
    }
  }
}

// Merge nsplit partial results per query row: grid = (B*Hkv*rows), block = LF_D.
extern "C" __global__ void __launch_bounds__(LF_HEAD_DIM) lf_attn_decode_combine(const LfAttnParams p) {
  const int d = threadIdx.x;
  const long long rowid = blockIdx.x;               // (bh * rows + qr)
  const int qr = (int)(rowid % p.rows);
  const int bh = (int)(rowid / p.rows);
  const int hkv = bh % p.Hkv;
  const int b = bh / p.Hkv;
  float m = LF_NEG_INF;
  for (int z = 0; z < p.nsplit; ++z) m = fmaxf(m, p.part_ml[(rowid * p.nsplit + z) * 2]);
  const float m_sub = (m == LF_NEG_INF) ? 0.0f : m;
  float l = 0.0f, a = 0.0f;
  for (int z = 0; z < p.nsplit; ++z) {
    const long long slot = rowid * p.nsplit + z;
    const float f = lf_exp2(p.part_ml[slot * 2] - m_sub);
    l += p.part_ml[slot * 2 + 1] * f;
    a += p.part_acc[slot * LF_HEAD_DIM + d] * f;
  }
  lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)hkv * p.o_sh + (long long)qr * p.o_ss;
  orow[d] = lf_from_float(a / l);
}
