// lf_attn_decode.hip — split-K decode attention for gfx950 (few query rows per
// (batch, kv head), long KV): an HBM-streaming kernel with both products on MFMA.
//
// A "unit" is one (batch, kv head, row chunk): up to 16 query rows that share
// every K/V fetch (GQA group rows, reference tests/benchmark.py:439-443).
// grid = (units, nsplit); a workgroup of LF_DW waves owns tokens
// [z*split_len, (z+1)*split_len) of its unit and deals them to its waves in pairs
// of 16-token steps.  Nothing is shared between waves until the final merge, so
// the streaming loop has no barrier.
//
// Per step a lane (c = lane%16, g = lane/16) loads, 16 bytes at a time and
// straight from global memory into registers, the pieces d = 32*j + 8*g .. +7 of
// K[token c] and V[token c] (paged: through the page table, ids fetched two pairs
// ahead -- reference loopfuse/codegen.py:738-872).  Four register stages keep two
// pairs (32 KB per wave) in flight.
//   S^T = K Q^T :  the K registers ARE the A operand of v_mfma_f32_16x16x32
//                  (row = token, k = d); Q^T (rows padded to 16) is the B operand.
//                  Lane (q = c, g) receives S^T[tokens 4g..4g+3][q].
//   softmax     :  per query column, with one exponent offset per column shared by
//                  the four lane groups; it may lag the running max by
//                  2^LF_LAZY_LOG2, so the cross-lane max and the rescale of O sit
//                  in a rarely taken wave-uniform branch.
//   O^T += V^T P^T: P^T of a PAIR of steps is, as held, a B operand (k = 32
//                  tokens); V goes through a wave-private LDS tile and comes back
//                  transposed (ds_read_b64_tr_b16) as the A operand (row = d).
// O^T lives in 4*D/16 accumulator registers per lane whatever the number of rows.
// At the end the LF_DW waves are merged through LDS with the (offset, sum, acc)
// log-sum-exp combine; with nsplit > 1 the workgroup writes its partial to
// scratch and lf_attn_decode_combine merges the splits.  With LF_HEADWAVE the
// waves do not share a head: each writes its own result or partial.  (Merging the
// splits inside the same launch, by the last split to arrive, was measured slower
// than the second launch: the device-scope fences or write-through stores it needs
// between XCDs cost more than the launch.)

#ifndef LF_DW
#define LF_DW 4              /* waves per workgroup */
#endif
#ifndef LF_LAZY_LOG2
#define LF_LAZY_LOG2 8       /* slack of the softmax exponent offset, log2 units */
#endif
#ifndef LF_HEADWAVE
#define LF_HEADWAVE 0        /* 1: the waves of a workgroup take LF_DW consecutive kv heads of one batch
                                element (same tokens) instead of sharing one head: with a token-major
                                page pool, where the heads of a token lie side by side, the workgroup
                                then reads whole pages front to back.  No merge between waves; every
                                wave writes its own result (nsplit == 1) or partial. */
#endif
#ifndef LF_ROWLOAD
#define LF_ROWLOAD 0         /* 1 (register-staged path, no score bias, K/V dense or in pages of a multiple of 16
                                tokens): a load instruction reads whole rows -- 64 / (D/8) tokens x D elements,
                                every 128-byte line in one piece -- with non-temporal loads, and K goes through a
                                wave-private LDS tile like V.  Lane (token c, 64-byte quarter) loads, which are the
                                MFMA operand layout, touch half a line per instruction; with non-temporal loads
                                they would fetch every line twice. */
#endif
#define LF_PSTRIDE (LF_HEADWAVE ? 1 : LF_DW)   /* distance between the pairs of steps of one wave */
#define LF_DT (LF_DW * 64)
#define LF_D LF_HEAD_DIM
#define LF_NJ (LF_D / 32)    /* 16-byte pieces of a row held by one lane = k-steps of QK^T */
#define LF_NDB (LF_D / 16)   /* 16-row blocks of O^T */
#define LF_QROWS 16          /* query rows one unit can hold (MFMA N) */
#define LF_OSTRIDE (LF_D + 4) /* floats per row of the merge buffer */

#ifndef LF_BIAS
#define LF_BIAS 0            /* 1: additive score bias [B, kv head, row, key] (8-byte aligned rows), e.g. a mask
                                tensor of 0 / -inf; travels with the K/V registers of its step */
#endif

struct LfDecStage {
  lf_u32x4 k[LF_NJ];
  lf_u32x4 v[LF_NJ];
#if LF_BIAS
  lf_elem4 bias;             // lane (q = c, g): keys 4g .. 4g + 3 of the step, query row q
#endif
};
struct LfDecIds {            // page ids of one step
  long long k, v;
};

#ifndef LF_COOP
#define LF_COOP 0            /* 1 (with LF_HEADWAVE, K and V paged, pages of a multiple of 16 tokens, token-major
                                pools): the workgroup loads each 16-token step of its LF_DW heads as ONE
                                contiguous block (16 token rows x LF_DW heads x D), every load instruction 1 KB
                                of consecutive bytes, and hands the rows to the waves through LDS.  Reading
                                the same bytes head by head -- 256-byte pieces 2 KB apart per wave -- costs
                                about a tenth of the HBM rate. */
#endif

#if LF_COOP
#if !LF_HEADWAVE || LF_PAGED != 3 || LF_BIAS || (LF_PAGE_SIZE % 16) || (LF_PAGE_SIZE_V % 16)
#error "LF_COOP needs LF_HEADWAVE, paged K and V with pages of a multiple of 16 tokens, and no score bias"
#endif

struct LfCoopStage {
  lf_u32x4 k[LF_NJ];
  lf_u32x4 v[LF_NJ];
};

// Split decode step, cooperative loads.  Layout of the work as in the kernel below with
// LF_HEADWAVE: grid = (B * Hkv/LF_DW, nsplit), wave w owns kv head LF_DW*hc + w and writes its
// own result or partial.  What differs is the way K and V reach the waves:
//   global -> registers : thread t of the workgroup loads 16-byte pieces t, t + LF_DT, ... of the
//                         step's block (LF_NJ pieces of K, LF_NJ of V); four steps in flight
//   registers -> LDS    : the same pieces, rows padded (K +16 B, V +32 B) so that the two read
//                         patterns below are free of bank conflicts; two buffers alternate,
//                         one workgroup barrier per step
//   LDS -> MFMA         : S^T = K Q^T with ds_read_b128 (row = token, 32 d per k-step) on the
//                         16x16x32 MFMA; O^T += V^T P^T with transposed 8-byte reads on the
//                         16x16x16 MFMA, whose k extent is the 16 tokens of a step
extern "C" __global__ void __launch_bounds__(LF_DT, 1) lf_attn_decode(const LfAttnParams p) {
  constexpr int kRowB = LF_DW * LF_D * 2;            // bytes of one token row over the workgroup's heads
  constexpr int kPieces = kRowB / 16;                // 16-byte pieces per row
  constexpr int kKStride = kRowB + 16;               // LDS row strides
  constexpr int kVStride = kRowB + 32;
  constexpr int kBufB = 16 * (kKStride + kVStride);
  static_assert(16 * kPieces == LF_NJ * LF_DT, "a step is LF_NJ pieces per thread");
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kBufB];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int c = lane & 15;      // token of a step (K rows) / query column (MFMA results)
  const int g = lane >> 4;

  const int z = blockIdx.y;
  const int chunks = (p.rows + LF_QROWS - 1) / LF_QROWS;   // row chunks per (b, kv head)
  const int unit = blockIdx.x;
  const int rc = unit % chunks;
  const int hchunks = p.Hkv / LF_DW;                        // the host checks Hkv % LF_DW == 0
  const int hkv0 = ((unit / chunks) % hchunks) * LF_DW;
  const int hkv = hkv0 + wave;
  const int b = unit / (chunks * hchunks);
  const int bh = b * p.Hkv + hkv;
  const int row0 = rc * LF_QROWS;
  const int nrows = min(p.rows - row0, LF_QROWS);

  const int tok_begin = z * p.split_len;
  const int tok_end = min(tok_begin + p.split_len, p.Sk);
  const int nsteps = (max(tok_end - tok_begin, 0) + 15) / 16;   // the same for every wave of the workgroup

  // ---- B operand of S^T = K Q^T: lane (q = c, g) holds Q[row0 + q][32*j + 8*g .. +7]
  lf_elem8 qb[LF_NJ];
  {
    const lf_elem* qrow = p.q + (long long)b * p.q_sb + (long long)hkv * p.q_sh +
                          (long long)(row0 + min(c, nrows - 1)) * p.q_ss;
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) {
      lf_u32x4 raw = *reinterpret_cast<const lf_u32x4*>(qrow + 32 * j + 8 * g);
      if (c >= nrows) raw = lf_u32x4{0u, 0u, 0u, 0u};
      qb[j] = __builtin_bit_cast(lf_elem8, raw);
    }
  }
#if LF_SOFTCAP
  const float sc_in = p.scale / p.softcap;
  const float cexp = LF_LOG2E;
#else
  const float cexp = p.scale * LF_LOG2E;
#endif

  lf_f32x4 o[LF_NDB];          // O^T: lane (q = c, g) holds d = 16*db + 4*g + i
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db) o[db] = lf_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  float mc = LF_NEG_INF;       // exponent offset of column q (same in all 4 lane groups)
  float l_part = 0.0f;         // this lane's share of the sum

  // ---- loads: piece u of this thread is piece tid + LF_DT*u of the step's block
  // Page ids: one register holds the ids of 32 steps (lane l: step l % 32 of the chunk, K for
  // l < 32, V for l >= 32), issue() picks its pair with v_readlane.  The next chunk's register
  // is loaded 32 steps ahead.  So the loop's only vector memory operations are the K/V loads:
  // these complete in order, and a table load consumed between them would make the wave wait
  // for every load in flight.
  auto load_ids = [&](int st0) -> lf_table_t {
    const int tok = min(tok_begin + 16 * (st0 + (lane & 31)), p.Sk - 1);   // steps past the end: the last page (never issued)
    return lane < 32 ? reinterpret_cast<const lf_table_t*>(p.k_table)[(long long)b * p.kt_stride + tok / LF_PAGE_SIZE]
                     : reinterpret_cast<const lf_table_t*>(p.v_table)[(long long)b * p.vt_stride + tok / LF_PAGE_SIZE_V];
  };
  lf_table_t ids_cur = load_ids(0), ids_nxt = load_ids(32);
  auto id_of = [&](int st, int which) -> long long {
    const int l = (st & 31) + 32 * which;
#if LF_TABLE_I64
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(ids_cur & 0xffffffffll), l);
    const int hi = __builtin_amdgcn_readlane((int)(ids_cur >> 32), l);
    return ((long long)hi << 32) | lo;
#else
    return (long long)__builtin_amdgcn_readlane(ids_cur, l);
#endif
  };
  auto issue = [&](LfCoopStage& sg, int st) {
    if ((st & 31) == 0 && st > 0) {       // next chunk of ids (workgroup-uniform)
      ids_cur = ids_nxt;
      ids_nxt = load_ids(st + 32);
    }
    const long long idk = id_of(st, 0), idv = id_of(st, 1);
    const int tok0 = tok_begin + 16 * st;
#pragma unroll
    for (int u = 0; u < LF_NJ; ++u) {
      const int piece = tid + LF_DT * u;
      const int tk = min(tok0 + piece / kPieces, p.Sk - 1);  // rows past Sk: clamped, masked later
      const int within = 8 * (piece % kPieces);              // elements
      // every byte is read once, whole lines at a time: streaming (non-temporal) loads
      sg.k[u] = __builtin_nontemporal_load(reinterpret_cast<const lf_u32x4*>(
          p.k + idk * p.k_sb + (long long)(tk % LF_PAGE_SIZE) * p.k_ss + (long long)hkv0 * p.k_sh + within));
      sg.v[u] = __builtin_nontemporal_load(reinterpret_cast<const lf_u32x4*>(
          p.v + idv * p.v_sb + (long long)(tk % LF_PAGE_SIZE_V) * p.v_ss + (long long)hkv0 * p.v_sh + within));
    }
  };
  auto to_lds = [&](const LfCoopStage& sg, int buf) {
    unsigned char* base = smem + buf * kBufB;
#pragma unroll
    for (int u = 0; u < LF_NJ; ++u) {
      const int piece = tid + LF_DT * u;
      const int tk = piece / kPieces, within = 16 * (piece % kPieces);
      *reinterpret_cast<lf_u32x4*>(base + tk * kKStride + within) = sg.k[u];
      *reinterpret_cast<lf_u32x4*>(base + 16 * kKStride + tk * kVStride + within) = sg.v[u];
    }
  };

  // ---- one step (16 tokens) of this wave's head out of LDS buffer `buf`
  auto consume = [&](int buf, int st) {
    const unsigned char* kb = smem + buf * kBufB + wave * (LF_D * 2);
    const unsigned char* vb = kb + 16 * kKStride;
    lf_f32x4 x4 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) {
      const lf_u32x4 kf = *reinterpret_cast<const lf_u32x4*>(kb + c * kKStride + 64 * j + 16 * g);
      x4 = lf_mfma16(__builtin_bit_cast(lf_elem8, kf), qb[j], x4);
    }
    // lane (q = c, g): x4[i] is token t0 + i
    const int t0 = tok_begin + 16 * st + 4 * g;
    float x[4];
    float mx = LF_NEG_INF;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float s = x4[i];
#if LF_SOFTCAP
      s = p.softcap * lf_tanh(s * sc_in);
#endif
      x[i] = (t0 + i < tok_end) ? s * cexp : LF_NEG_INF;
      mx = fmaxf(mx, x[i]);
    }
    if (__builtin_amdgcn_ballot_w64(mx > mc + (float)LF_LAZY_LOG2) != 0ull) {
      // bring the column's offset up to its max over all four lane groups
      float mq = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mq = fmaxf(mq, __shfl_xor(mq, 32, 64));
      const float m_new = fmaxf(mc, mq);
      const float r = (m_new == LF_NEG_INF) ? 1.0f : lf_exp2(mc - m_new);
      mc = m_new;
      l_part *= r;
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db) o[db] *= r;
    }
    const float m_sub = (mc == LF_NEG_INF) ? 0.0f : mc;
    lf_elem4 pb;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float e = lf_exp2(x[i] - m_sub);
      l_part += e;
      pb[i] = lf_from_float(e);
    }
    // O^T += V^T P^T: k-slot i of lane group g is token 4g + i, the order pb is held in.  The
    // 16 lanes of a group ask for rows 4g .. 4g+3, columns 16db .. +15: lane c supplies the
    // 8-byte piece (row 4g + c/4, columns +4*(c%4)) and receives column c of the four rows.
    const int trow = 4 * g + (c >> 2);
#pragma unroll
    for (int db = 0; db < LF_NDB; ++db) {
      const unsigned char* src = vb + trow * kVStride + 2 * (16 * db + 4 * (c & 3));
      lf_s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(src));
      o[db] = lf_mfma16k16(__builtin_bit_cast(lf_elem4, t), pb, o[db]);
    }
  };

  // ---- streaming loop: four register stages rotate (static names: four steps per trip)
  {
    LfCoopStage s0, s1, s2, s3;
    // step st: stage -> LDS buffer st & 1, refill the stage with step st + 4, barrier (LDS
    // writes only: the loads stay in flight), consume.  Buffer st & 1 was last read in step
    // st - 2, which every wave had left before it arrived at the barrier of step st - 1.
#define LF_COOP_STEP(sg, st, refill)                                         \
    {                                                                        \
      to_lds(sg, (st) & 1);                                                  \
      if (refill) issue(sg, (st) + 4);                                       \
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");        \
      consume((st) & 1, (st));                                               \
    }
    // The steady state has no condition in it: the compiler counts the loads in flight to
    // place its waits, and a path on which a refill is skipped would make it wait, on every
    // path, as if the stage being written were the last one loaded (i.e. for everything).
    int st = 0;
    if (nsteps >= 8) {
      issue(s0, 0);
      issue(s1, 1);
      issue(s2, 2);
      issue(s3, 3);
      do {
        LF_COOP_STEP(s0, st, true)
        LF_COOP_STEP(s1, st + 1, true)
        LF_COOP_STEP(s2, st + 2, true)
        LF_COOP_STEP(s3, st + 3, true)
        st += 4;
      } while (st + 8 <= nsteps);
    } else {
      if (0 < nsteps) issue(s0, 0);
      if (1 < nsteps) issue(s1, 1);
      if (2 < nsteps) issue(s2, 2);
      if (3 < nsteps) issue(s3, 3);
    }
    for (; st < nsteps; st += 4) {
      if (st < nsteps) LF_COOP_STEP(s0, st, st + 4 < nsteps)
      if (st + 1 < nsteps) LF_COOP_STEP(s1, st + 1, st + 5 < nsteps)
      if (st + 2 < nsteps) LF_COOP_STEP(s2, st + 2, st + 6 < nsteps)
      if (st + 3 < nsteps) LF_COOP_STEP(s3, st + 3, st + 7 < nsteps)
    }
#undef LF_COOP_STEP
  }

  // ---- every wave owns its (batch, head): lane (q = c, g) writes d = 16*db + 4*g .. +3 of row q
  float l_wave = l_part + __shfl_xor(l_part, 16, 64);
  l_wave += __shfl_xor(l_wave, 32, 64);
  if (c < nrows) {
    const int qr = row0 + c;
    if (p.nsplit == 1) {
      lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)hkv * p.o_sh + (long long)qr * p.o_ss;
      const float inv = lf_inv_sum(l_wave);
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db) {
        lf_elem4 w4;
#pragma unroll
        for (int e = 0; e < 4; ++e) w4[e] = lf_from_float(o[db][e] * inv);
        *reinterpret_cast<lf_elem4*>(orow + 16 * db + 4 * g) = w4;
      }
    } else {
      const long long slot = ((long long)bh * p.rows + qr) * p.nsplit + z;
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db)
        *reinterpret_cast<lf_f32x4*>(&p.part_acc[slot * LF_D + 16 * db + 4 * g]) = o[db];
      if (g == 0) {
        p.part_ml[slot * 2 + 0] = mc;            // exponent offset, log2 units
        p.part_ml[slot * 2 + 1] = l_wave;
      }
    }
  }
}
#else   // !LF_COOP
extern "C" __global__ void __launch_bounds__(LF_DT, 8 / LF_DW) lf_attn_decode(const LfAttnParams p) {
  // One buffer, two lives: wave-private V tiles of the pair being consumed
  // ([LF_DW][2][16*D] elements) during the loop, merge buffer
  // ([LF_DW][16][LF_OSTRIDE] floats) after it.
  constexpr int kVBytes = LF_DW * 2 * 16 * LF_D * 2 * (LF_ROWLOAD ? 2 : 1);   // wave-private V (and K) tiles of a pair
  constexpr int kOBytes = LF_DW * LF_QROWS * LF_OSTRIDE * 4;
  __shared__ __attribute__((aligned(16))) unsigned char smem[kVBytes > kOBytes ? kVBytes : kOBytes];
#if !LF_HEADWAVE
  __shared__ float red_m[LF_DW][LF_QROWS];
  __shared__ float red_l[LF_DW][LF_QROWS];
#endif

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int c = lane & 15;      // token of a step (loads) / query column (MFMA results)
  const int g = lane >> 4;

  const int z = blockIdx.y;
  const int chunks = (p.rows + LF_QROWS - 1) / LF_QROWS;   // row chunks per (b, kv head)
  const int unit = blockIdx.x;
  const int rc = unit % chunks;
#if LF_HEADWAVE
  // grid.x = B * ceil(Hkv / LF_DW) * chunks; wave w serves head LF_DW*hc + w
  const int hchunks = (p.Hkv + LF_DW - 1) / LF_DW;
  const int hkv = ((unit / chunks) % hchunks) * LF_DW + wave;
  const int b = unit / (chunks * hchunks);
  if (hkv >= p.Hkv) return;          // no workgroup barrier in this mode
  const int bh = b * p.Hkv + hkv;
#else
  const int bh = unit / chunks;
  const int hkv = bh % p.Hkv;
  const int b = bh / p.Hkv;
#endif
  const int row0 = rc * LF_QROWS;
  const int nrows = min(p.rows - row0, LF_QROWS);          // query rows of this unit

  int tok_begin = z * p.split_len;
  int tok_end = min(tok_begin + p.split_len, p.Sk);
#if LF_BIAS
  // Keys whose bias is -inf for every query row of the unit add nothing.  The split is narrowed
  // to the span from its first to its last live key (the left padding of a batch, the unused
  // tail of a fixed-size cache are then never read); a split without a live key does no work.
  // Every wave scans the same values (4 keys per lane, 256 per step) and finds the same span.
  {
    const lf_elem* bb = p.bias + (long long)b * p.bias_sb + (long long)hkv * p.bias_sh + (long long)row0 * p.bias_sq;
    const int nscan = p.bias_sq == 0 ? 1 : nrows;       // rows that share one bias row are scanned once
    int first = 0x7fffffff, last = -1;                  // relative to tok_begin
    for (int base = tok_begin; base < tok_end; base += 256) {
      const int t4 = base + 4 * lane;
      bool lv = false;
      for (int r = 0; r < nscan; ++r) {
        const lf_elem* br = bb + (long long)r * p.bias_sq;
        if (t4 + 3 < tok_end) {
          const lf_u32x2 raw = *reinterpret_cast<const lf_u32x2*>(br + t4);
          lv = lv || !lf_bias_masked2(raw[0]) || !lf_bias_masked2(raw[1]);
        } else {
          for (int e = 0; e < 4; ++e)
            if (t4 + e < tok_end) lv = lv || !lf_bias_masked(__builtin_bit_cast(unsigned short, br[t4 + e]));
        }
      }
      const unsigned long long live = __builtin_amdgcn_ballot_w64(lv);
      if (live != 0ull) {
        first = min(first, base - tok_begin + 4 * (int)__builtin_ctzll(live));
        last = max(last, base - tok_begin + 4 * (63 - (int)__builtin_clzll(live)) + 3);
      }
    }
    if (last < 0) {
      tok_end = tok_begin;
    } else {
      tok_end = min(tok_end, tok_begin + last + 1);
      tok_begin += first & ~31;                         // whole pairs of 16-key steps
    }
  }
#endif
  const int npairs = (max(tok_end - tok_begin, 0) + 31) / 32;

  // ---- B operand of S^T = K Q^T: lane (q = c, g) holds Q[row0 + q][32*j + 8*g .. +7];
  // columns past nrows are zero
  lf_elem8 qb[LF_NJ];
  {
    const lf_elem* qrow = p.q + (long long)b * p.q_sb + (long long)hkv * p.q_sh +
                          (long long)(row0 + min(c, nrows - 1)) * p.q_ss;
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) {
      lf_u32x4 raw = *reinterpret_cast<const lf_u32x4*>(qrow + 32 * j + 8 * g);
      if (c >= nrows) raw = lf_u32x4{0u, 0u, 0u, 0u};
      qb[j] = __builtin_bit_cast(lf_elem8, raw);
    }
  }

#if LF_SOFTCAP
  const float sc_in = p.scale / p.softcap;
  const float cexp = LF_LOG2E;
#else
  const float cexp = p.scale * LF_LOG2E;
#endif

  lf_f32x4 o[LF_NDB];          // O^T: lane (q = c, g) holds d = 16*db + 4*g + i
#pragma unroll
  for (int db = 0; db < LF_NDB; ++db) o[db] = lf_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  float mc = LF_NEG_INF;       // exponent offset of column q (same in all 4 lane groups)
  float l_part = 0.0f;         // this lane's share of the sum

  // ---- addressing
  constexpr bool kPagedK = (LF_PAGED & 1) != 0;
  constexpr bool kPagedV = (LF_PAGED & 2) != 0;
  // pages of >= 16 tokens: a 16-token step lies inside one page, the id is wave-uniform
  constexpr bool kUniformPage = (!kPagedK || (LF_PAGE_SIZE % 16) == 0) && (!kPagedV || (LF_PAGE_SIZE_V % 16) == 0);
  auto step_tok0 = [&](int st) { return tok_begin + 16 * st; };
  auto fetch_ids = [&](int st) {
    LfDecIds id = {0, 0};
    if (kPagedK || kPagedV) {
      // clamp: steps past the end re-read the last page (their scores are masked)
      const int tok = min(step_tok0(st) + (kUniformPage ? 0 : c), p.Sk - 1);
      if (kPagedK) id.k = reinterpret_cast<const lf_table_t*>(p.k_table)[(long long)b * p.kt_stride + tok / LF_PAGE_SIZE];
      if (kPagedV) id.v = reinterpret_cast<const lf_table_t*>(p.v_table)[(long long)b * p.vt_stride + tok / LF_PAGE_SIZE_V];
    }
    return id;
  };
#if LF_BIAS
  // bias row of query column c (columns past nrows repeat the last row; their results are dropped)
  const lf_elem* bias_row = p.bias + (long long)b * p.bias_sb + (long long)hkv * p.bias_sh +
                            (long long)(row0 + min(c, nrows - 1)) * p.bias_sq;
#endif
  auto issue = [&](LfDecStage& sg, int st, const LfDecIds& id) {
#if LF_ROWLOAD
    // load u of the step: tokens kTokPerLoad*u .. +kTokPerLoad-1, lane = (token, 16-byte piece of its row)
    constexpr int kCpr = LF_D / 8, kTokPerLoad = 64 / kCpr;
    static_assert(kTokPerLoad * LF_NJ == 16, "LF_NJ loads cover the 16 tokens of a step");
    const int lt = lane / kCpr, piece = lane % kCpr;
#pragma unroll
    for (int u = 0; u < LF_NJ; ++u) {
      const int tok = min(step_tok0(st) + kTokPerLoad * u + lt, p.Sk - 1);   // clamp: masked later, never out of bounds
      const lf_elem *kp, *vp;
      if (kPagedK)
        kp = p.k + id.k * p.k_sb + (long long)(tok % LF_PAGE_SIZE) * p.k_ss + (long long)hkv * p.k_sh;
      else
        kp = p.k + (long long)b * p.k_sb + (long long)hkv * p.k_sh + (long long)tok * p.k_ss;
      if (kPagedV)
        vp = p.v + id.v * p.v_sb + (long long)(tok % LF_PAGE_SIZE_V) * p.v_ss + (long long)hkv * p.v_sh;
      else
        vp = p.v + (long long)b * p.v_sb + (long long)hkv * p.v_sh + (long long)tok * p.v_ss;
      sg.k[u] = __builtin_nontemporal_load(reinterpret_cast<const lf_u32x4*>(kp + 8 * piece));
      sg.v[u] = __builtin_nontemporal_load(reinterpret_cast<const lf_u32x4*>(vp + 8 * piece));
    }
#else
    const int tok = min(step_tok0(st) + c, p.Sk - 1);      // clamp: masked later, never out of bounds
    const lf_elem *kp, *vp;
    if (kPagedK)
      kp = p.k + id.k * p.k_sb + (long long)(tok % LF_PAGE_SIZE) * p.k_ss + (long long)hkv * p.k_sh + 8 * g;
    else
      kp = p.k + (long long)b * p.k_sb + (long long)hkv * p.k_sh + (long long)tok * p.k_ss + 8 * g;
    if (kPagedV)
      vp = p.v + id.v * p.v_sb + (long long)(tok % LF_PAGE_SIZE_V) * p.v_ss + (long long)hkv * p.v_sh + 8 * g;
    else
      vp = p.v + (long long)b * p.v_sb + (long long)hkv * p.v_sh + (long long)tok * p.v_ss + 8 * g;
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) sg.k[j] = *reinterpret_cast<const lf_u32x4*>(kp + 32 * j);
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) sg.v[j] = *reinterpret_cast<const lf_u32x4*>(vp + 32 * j);
#endif
#if LF_BIAS
    {
      // keys past Sk read clamped positions: their scores are masked in consume()
      const int t4 = step_tok0(st) + 4 * g;
      if (t4 + 3 < p.Sk) {
        sg.bias = *reinterpret_cast<const lf_elem4*>(bias_row + t4);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) sg.bias[e] = bias_row[min(t4 + e, p.Sk - 1)];
      }
    }
#endif
  };

  lf_elem* my_v = reinterpret_cast<lf_elem*>(smem) + wave * 2 * 16 * LF_D * (LF_ROWLOAD ? 2 : 1);
#if LF_ROWLOAD
  lf_elem* my_k = my_v + 2 * 16 * LF_D;
  // rows as loaded -> the wave-private tiles of step hsel: V with the chunk swizzle of the
  // transposed reads below, K with chunk ^ (row & (chunks - 1)) so that the 16 rows one
  // ds_read_b128 of a fragment touches lie on different banks
  auto stash_kv = [&](const LfDecStage& sg, int hsel) {
    constexpr int kCpr = LF_D / 8, kTokPerLoad = 64 / kCpr;
    const int lt = lane / kCpr, piece = lane % kCpr;
#pragma unroll
    for (int u = 0; u < LF_NJ; ++u) {
      const int row = kTokPerLoad * u + lt;
      *reinterpret_cast<lf_u32x4*>(&my_v[hsel * 16 * LF_D + row * LF_D + 8 * (piece ^ (2 * (row & 3)))]) = sg.v[u];
      *reinterpret_cast<lf_u32x4*>(&my_k[hsel * 16 * LF_D + row * LF_D + 8 * (piece ^ (row & (kCpr - 1)))]) = sg.k[u];
    }
  };
  auto k_frag = [&](int hsel, int j) {      // A operand of k-step j: lane (token c, g) holds d = 32 j + 8 g .. +7
    constexpr int kCpr = LF_D / 8;
    return *reinterpret_cast<const lf_u32x4*>(&my_k[hsel * 16 * LF_D + c * LF_D + 8 * ((4 * j + g) ^ (c & (kCpr - 1)))]);
  };
#endif
  // V rows of a step -> wave-private LDS tile hsel (row = token c, 16-byte chunk
  // 4j+g, chunk index XORed with 2*(row&3) so that the 4 rows a transposed read
  // touches sit on different banks)
  auto stash_v = [&](const LfDecStage& sg, int hsel) {
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) {
      const int ch = (4 * j + g) ^ (2 * (c & 3));
      *reinterpret_cast<lf_u32x4*>(&my_v[hsel * 16 * LF_D + c * LF_D + 8 * ch]) = sg.v[j];
    }
  };

  // ---- one pair of steps (32 tokens)
  auto consume = [&](const LfDecStage& sa, const LfDecStage& sb, int pr) {
    lf_f32x4 xa = {0.0f, 0.0f, 0.0f, 0.0f}, xb = {0.0f, 0.0f, 0.0f, 0.0f};
#if LF_ROWLOAD
    stash_kv(sa, 0);
    stash_kv(sb, 1);
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) {
      xa = lf_mfma16(__builtin_bit_cast(lf_elem8, k_frag(0, j)), qb[j], xa);
      xb = lf_mfma16(__builtin_bit_cast(lf_elem8, k_frag(1, j)), qb[j], xb);
    }
#else
#pragma unroll
    for (int j = 0; j < LF_NJ; ++j) {
      xa = lf_mfma16(__builtin_bit_cast(lf_elem8, sa.k[j]), qb[j], xa);
      xb = lf_mfma16(__builtin_bit_cast(lf_elem8, sb.k[j]), qb[j], xb);
    }
    stash_v(sa, 0);
    stash_v(sb, 1);
#endif

    // lane (q = c, g): xa[i] is token t0 + i, xb[i] token t0 + 16 + i
    const int t0 = step_tok0(2 * pr) + 4 * g;
    float x[8];
    float mx = LF_NEG_INF;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float s = (i < 4) ? xa[i] : xb[i - 4];
#if LF_SOFTCAP
      s = p.softcap * lf_tanh(s * sc_in);
#endif
      const int tok = t0 + (i < 4 ? i : 12 + i);
#if LF_BIAS
      // (scaled or capped score + bias) in log2 units
      x[i] = (tok < tok_end) ? s * cexp + lf_bias_value(i < 4 ? sa.bias[i] : sb.bias[i - 4]) * LF_LOG2E : LF_NEG_INF;
#else
      x[i] = (tok < tok_end) ? s * cexp : LF_NEG_INF;
#endif
      mx = fmaxf(mx, x[i]);
    }
    if (__builtin_amdgcn_ballot_w64(mx > mc + (float)LF_LAZY_LOG2) != 0ull) {
      // bring the column's offset up to its max over all four lane groups
      float mq = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mq = fmaxf(mq, __shfl_xor(mq, 32, 64));
      const float m_new = fmaxf(mc, mq);
      const float r = (m_new == LF_NEG_INF) ? 1.0f : lf_exp2(mc - m_new);
      mc = m_new;
      l_part *= r;
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db) o[db] *= r;
    }
    const float m_sub = (mc == LF_NEG_INF) ? 0.0f : mc;
    lf_elem8 pb;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float e = lf_exp2(x[i] - m_sub);
      l_part += e;
      pb[i] = lf_from_float(e);
    }

    // O^T += V^T P^T: k-slot s of lane group g is token 4g + s (s < 4) of the first
    // step and 4g + s - 4 of the second -- the order pb is held in
    const int trow = 4 * g + (c >> 2);          // row this lane addresses for its 16-lane group
#pragma unroll
    for (int db = 0; db < LF_NDB; ++db) {
      const int col = 16 * db + 4 * (c & 3);
      const int ch = (col / 8) ^ (2 * (trow & 3));
      lf_elem8 a;
#pragma unroll
      for (int hsel = 0; hsel < 2; ++hsel) {
        const lf_elem* src = &my_v[hsel * 16 * LF_D + trow * LF_D + 8 * ch + (col % 8)];
        lf_s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(src));
        lf_elem4 te = __builtin_bit_cast(lf_elem4, t);
        a[4 * hsel + 0] = te[0];
        a[4 * hsel + 1] = te[1];
        a[4 * hsel + 2] = te[2];
        a[4 * hsel + 3] = te[3];
      }
      o[db] = lf_mfma16(a, pb, o[db]);
    }
  };

  // ---- streaming loop: this wave's pairs are wave, wave + LF_DW, ... (all pairs of the
  // split when each wave has its own head); four register
  // stages (two pairs) rotate, two trips of the pipeline per loop iteration so every
  // stage has a static name
  {
    LfDecStage s0, s1, s2, s3;
    LfDecIds i0, i1, i2, i3;
    int pr = LF_HEADWAVE ? 0 : wave;
    i0 = fetch_ids(2 * pr);
    i1 = fetch_ids(2 * pr + 1);
    i2 = fetch_ids(2 * (pr + LF_PSTRIDE));
    i3 = fetch_ids(2 * (pr + LF_PSTRIDE) + 1);
    // The steady state (both pairs of the trip and both refills exist) has no condition in it:
    // the compiler places its waits by counting the loads in flight, and a path on which a
    // refill is skipped would make it wait on every path as if nothing younger were in flight,
    // i.e. for all loads.  The last trips run below, with the conditions.
    if (pr + 3 * LF_PSTRIDE < npairs) {
      issue(s0, 2 * pr, i0);
      issue(s1, 2 * pr + 1, i1);
      i0 = fetch_ids(2 * (pr + 2 * LF_PSTRIDE));
      i1 = fetch_ids(2 * (pr + 2 * LF_PSTRIDE) + 1);
      issue(s2, 2 * (pr + LF_PSTRIDE), i2);
      issue(s3, 2 * (pr + LF_PSTRIDE) + 1, i3);
      i2 = fetch_ids(2 * (pr + 3 * LF_PSTRIDE));
      i3 = fetch_ids(2 * (pr + 3 * LF_PSTRIDE) + 1);
      do {
        consume(s0, s1, pr);
        const int pa = pr + 2 * LF_PSTRIDE;
        issue(s0, 2 * pa, i0);
        issue(s1, 2 * pa + 1, i1);
        i0 = fetch_ids(2 * (pa + 2 * LF_PSTRIDE));
        i1 = fetch_ids(2 * (pa + 2 * LF_PSTRIDE) + 1);
        const int pb2 = pr + LF_PSTRIDE;
        consume(s2, s3, pb2);
        const int pc = pb2 + 2 * LF_PSTRIDE;
        issue(s2, 2 * pc, i2);
        issue(s3, 2 * pc + 1, i3);
        i2 = fetch_ids(2 * (pc + 2 * LF_PSTRIDE));
        i3 = fetch_ids(2 * (pc + 2 * LF_PSTRIDE) + 1);
        pr += 2 * LF_PSTRIDE;
      } while (pr + 3 * LF_PSTRIDE < npairs);
    } else {
      if (pr < npairs) {
        issue(s0, 2 * pr, i0);
        issue(s1, 2 * pr + 1, i1);
        i0 = fetch_ids(2 * (pr + 2 * LF_PSTRIDE));
        i1 = fetch_ids(2 * (pr + 2 * LF_PSTRIDE) + 1);
      }
      if (pr + LF_PSTRIDE < npairs) {
        issue(s2, 2 * (pr + LF_PSTRIDE), i2);
        issue(s3, 2 * (pr + LF_PSTRIDE) + 1, i3);
        i2 = fetch_ids(2 * (pr + 3 * LF_PSTRIDE));
        i3 = fetch_ids(2 * (pr + 3 * LF_PSTRIDE) + 1);
      }
    }
    for (; pr < npairs; pr += 2 * LF_PSTRIDE) {
      consume(s0, s1, pr);
      const int pa = pr + 2 * LF_PSTRIDE;
      if (pa < npairs) {
        issue(s0, 2 * pa, i0);
        issue(s1, 2 * pa + 1, i1);
        i0 = fetch_ids(2 * (pa + 2 * LF_PSTRIDE));
        i1 = fetch_ids(2 * (pa + 2 * LF_PSTRIDE) + 1);
      }
      const int pb2 = pr + LF_PSTRIDE;
      if (pb2 < npairs) {
        consume(s2, s3, pb2);
        const int pc = pb2 + 2 * LF_PSTRIDE;
        if (pc < npairs) {
          issue(s2, 2 * pc, i2);
          issue(s3, 2 * pc + 1, i3);
          i2 = fetch_ids(2 * (pc + 2 * LF_PSTRIDE));
          i3 = fetch_ids(2 * (pc + 2 * LF_PSTRIDE) + 1);
        }
      }
    }
  }

  // ---- merge: lane groups (sum), then the LF_DW waves
  float l_wave = l_part + __shfl_xor(l_part, 16, 64);
  l_wave += __shfl_xor(l_wave, 32, 64);
#if LF_HEADWAVE
  // each wave owns its (batch, head): lane (q = c, g) writes d = 16*db + 4*g .. +3 of row q
  if (c < nrows) {
    const int qr = row0 + c;
    if (p.nsplit == 1) {
      lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)hkv * p.o_sh + (long long)qr * p.o_ss;
      const float inv = lf_inv_sum(l_wave);
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db) {
        lf_elem4 w4;
#pragma unroll
        for (int e = 0; e < 4; ++e) w4[e] = lf_from_float(o[db][e] * inv);
        *reinterpret_cast<lf_elem4*>(orow + 16 * db + 4 * g) = w4;
      }
    } else {
      const long long slot = ((long long)bh * p.rows + qr) * p.nsplit + z;
#pragma unroll
      for (int db = 0; db < LF_NDB; ++db)
        *reinterpret_cast<lf_f32x4*>(&p.part_acc[slot * LF_D + 16 * db + 4 * g]) = o[db];
      if (g == 0) {
        p.part_ml[slot * 2 + 0] = mc;            // exponent offset, log2 units
        p.part_ml[slot * 2 + 1] = l_wave;
      }
    }
  }
#else
  if (g == 0) {
    red_m[wave][c] = mc;
    red_l[wave][c] = l_wave;
  }
  __syncthreads();   // also: every wave is done with its V tiles, smem changes role
  float* red_o = reinterpret_cast<float*>(smem);
  {
    float m_wg = red_m[0][c];
#pragma unroll
    for (int w = 1; w < LF_DW; ++w) m_wg = fmaxf(m_wg, red_m[w][c]);
    const float m_sub = (m_wg == LF_NEG_INF) ? 0.0f : m_wg;
    const float f = lf_exp2(mc - m_sub);        // 0 for a wave that saw nothing
#pragma unroll
    for (int db = 0; db < LF_NDB; ++db)
      *reinterpret_cast<lf_f32x4*>(&red_o[(wave * LF_QROWS + c) * LF_OSTRIDE + 16 * db + 4 * g]) = o[db] * f;
  }
  __syncthreads();
  // thread -> (query row qi, 8 consecutive d's)
  for (int item = tid; item < LF_QROWS * LF_D / 8; item += LF_DT) {
    const int qi = item / (LF_D / 8);
    const int d0 = (item % (LF_D / 8)) * 8;
    if (qi >= nrows) continue;
    float m_all = red_m[0][qi];
#pragma unroll
    for (int w = 1; w < LF_DW; ++w) m_all = fmaxf(m_all, red_m[w][qi]);
    const float ms = (m_all == LF_NEG_INF) ? 0.0f : m_all;
    float l_tot = 0.0f;
#pragma unroll
    for (int w = 0; w < LF_DW; ++w) l_tot += red_l[w][qi] * lf_exp2(red_m[w][qi] - ms);
    float sum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = 0.0f;
#pragma unroll
    for (int w = 0; w < LF_DW; ++w)
#pragma unroll
      for (int e = 0; e < 8; ++e) sum[e] += red_o[(w * LF_QROWS + qi) * LF_OSTRIDE + d0 + e];
    const int qr = row0 + qi;
    if (p.nsplit == 1) {
      lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)hkv * p.o_sh + (long long)qr * p.o_ss;
      const float inv = lf_inv_sum(l_tot);
      lf_elem8 w8;
#pragma unroll
      for (int e = 0; e < 8; ++e) w8[e] = lf_from_float(sum[e] * inv);
      *reinterpret_cast<lf_elem8*>(orow + d0) = w8;
    } else {
      const long long slot = ((long long)bh * p.rows + qr) * p.nsplit + z;
#pragma unroll
      for (int e = 0; e < 8; ++e) p.part_acc[slot * LF_D + d0 + e] = sum[e];
      if (d0 == 0) {
        p.part_ml[slot * 2 + 0] = m_all;       // exponent offset, log2 units
        p.part_ml[slot * 2 + 1] = l_tot;
      }
    }
  }
#endif   // LF_HEADWAVE
}

#endif  // LF_COOP

// Merge nsplit partial results per query row.  A thread owns 4 consecutive d of one row;
// block = 256 threads = 1024 / LF_HEAD_DIM rows, grid = ceil(B*Hkv*rows / rows per block).
extern "C" __global__ void __launch_bounds__(256) lf_attn_decode_combine(const LfAttnParams p) {
  constexpr int kTPR = LF_HEAD_DIM / 4;              // threads per row
  constexpr int kRPB = 256 / kTPR;                   // rows per block
  const long long rowid = (long long)blockIdx.x * kRPB + threadIdx.x / kTPR;   // (bh * rows + qr)
  const long long nrows = (long long)p.B * p.Hkv * p.rows;
  if (rowid >= nrows) return;
  const int d0 = 4 * (threadIdx.x % kTPR);
  const int qr = (int)(rowid % p.rows);
  const int bh = (int)(rowid / p.rows);
  const int hkv = bh % p.Hkv;
  const int b = bh / p.Hkv;
  // four splits at a time: their eight loads are issued together (one memory round trip
  // per group instead of one per split), then merged into the running (offset, sum, acc)
  float m = LF_NEG_INF;
  float l = 0.0f;
  lf_f32x4 a = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int z0 = 0; z0 < p.nsplit; z0 += 4) {
    lf_f32x2 ml[4];
    lf_f32x4 ac[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const long long slot = rowid * p.nsplit + min(z0 + u, p.nsplit - 1);
      ml[u] = *reinterpret_cast<const lf_f32x2*>(&p.part_ml[slot * 2]);
      ac[u] = *reinterpret_cast<const lf_f32x4*>(&p.part_acc[slot * LF_HEAD_DIM + d0]);
    }
    float mc = m;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (z0 + u < p.nsplit) mc = fmaxf(mc, ml[u][0]);
    const float m_sub = (mc == LF_NEG_INF) ? 0.0f : mc;
    const float r = (m == LF_NEG_INF) ? 0.0f : lf_exp2(m - m_sub);   // nothing merged yet: l and a are 0
    l *= r;
    a *= r;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (z0 + u < p.nsplit) {
        const float f = lf_exp2(ml[u][0] - m_sub);
        l += ml[u][1] * f;
        a += ac[u] * f;
      }
    m = mc;
  }
  lf_elem* orow = p.o + (long long)b * p.o_sb + (long long)hkv * p.o_sh + (long long)qr * p.o_ss;
  const float inv = lf_inv_sum(l);
  lf_elem4 w;
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] = lf_from_float(a[e] * inv);
  *reinterpret_cast<lf_elem4*>(orow + d0) = w;
}
