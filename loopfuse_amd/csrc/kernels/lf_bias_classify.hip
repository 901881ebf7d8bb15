// lf_bias_classify.hip — tile classes of an additive score bias, for lf_attn_prefill_swp -DLF_BIAS=1.
//
// Mask tensors reach the kernels as score biases of 0 / -inf (attn_mask of
// F.scaled_dot_product_attention, hand-written `scores + mask`, boolean masks turned into
// that form by the front end).  Most (q tile, kv tile) blocks of such a bias are all -inf
// (nothing of the block is visible: the attention kernel does not compute it, and does not
// walk it at either end of a q tile's range) or all zero (the block needs no bias at all);
// only the few blocks on the edge of the visible region mix values.  This kernel reads the
// bias once per distinct (batch, head) it holds and writes, per q tile (128 rows; 64 or 32 when the
// attention kernel packs query heads, which it does only for a bias shared by all heads) and kv
// tile of 64 keys,
//
//   class[unit][kv tile] = 0 dead | 1 zero | 2 mixed                (int32)
//
// into p.part_acc, unit = (batch' * heads' + head') * q_tiles + q_tile with batch' / head'
// collapsed to 0 where the bias is broadcast (stride 0).
// A dense bias of real numbers costs two loads per block: only blocks whose bottom-left and
// top-right corners are both masked, or both zero, are read in full.
//
// Grid (q tiles, batches' * heads', groups of 4 kv tiles), 256 threads: one wave per block,
// 32 eight-byte loads per lane, all in flight together.  Needs bias rows that start on 8-byte
// boundaries (p.bias_sq and the strides multiples of 4) and Sk >= 4.
//
// The reference has no counterpart: its mask ops are index predicates
// (loopfuse/torch_backend/ops.py:675-751) and a mask given as data is not skipped over.

#define LF_BC_BM LF_BM      /* rows of the attention kernel's q tile: 128, or 64 / 32 with packed query heads */
#define LF_BC_BN LF_BN

extern "C" __global__ __launch_bounds__(256) void lf_bias_classify(const LfAttnParams p) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nqt = (p.Sq + LF_BC_BM - 1) / LF_BC_BM;
  const int nkt = (p.Sk + LF_BC_BN - 1) / LF_BC_BN;
  const int nhh = p.bias_sh ? p.Hq : 1;
  const int qt = blockIdx.x;
  const int bb = blockIdx.y / nhh, hh = blockIdx.y % nhh;
  const int unit = (bb * nhh + hh) * nqt + qt;
  const int kt = 4 * blockIdx.z + wave;
  if (kt >= nkt) return;
  int* cls = reinterpret_cast<int*>(p.part_acc) + (long long)unit * nkt;
  const lf_elem* base = p.bias + (long long)bb * p.bias_sb + (long long)hh * p.bias_sh;
  const int q0 = qt * LF_BC_BM;
  const int qlast = min(q0 + LF_BC_BM, p.Sq) - 1;
  const int k0 = kt * LF_BC_BN;
  const int klast = min(k0 + LF_BC_BN, p.Sk) - 1;
  auto bits = [&](int q, int j) { return (unsigned)__builtin_bit_cast(unsigned short, base[(long long)q * p.bias_sq + j]); };
  auto is_zero = [](unsigned b16) { return (b16 & 0x7fffu) == 0u; };

  // candidates by two corners (wave-uniform values: every lane reads the same two elements)
  const unsigned bl = bits(qlast, k0), tr = bits(q0, klast);
  bool dead = lf_bias_masked(bl) && lf_bias_masked(tr);
  bool zero = is_zero(bl) && is_zero(tr);
  if (dead || zero) {
    // lane = (row in a group of 4, 4-key chunk): 8-byte loads, LF_BC_BM / 4 groups of 4 rows cover the tile
    const int j = k0 + 4 * (lane & 15), r4 = lane >> 4;
    const bool whole = j + 3 <= klast;
    const int jload = min(j, p.Sk - 4);        // the chunk that would run past Sk is read from Sk - 4 (and not used)
    // all loads of the lane go out before the first is looked at: one memory latency per block
    lf_u32x2 w[LF_BC_BM / 4];
#pragma unroll
    for (int u = 0; u < LF_BC_BM / 4; ++u) {
      const int q = min(q0 + 4 * u + r4, qlast);      // rows past the end re-read the last one
      w[u] = *reinterpret_cast<const lf_u32x2*>(base + (long long)q * p.bias_sq + jload);
    }
    if (whole) {
#pragma unroll
      for (int u = 0; u < LF_BC_BM / 4; ++u)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          dead = dead && lf_bias_masked2(w[u][e]);
          zero = zero && is_zero(w[u][e] & 0xffffu) && is_zero(w[u][e] >> 16);
        }
    } else if (j <= klast) {
      // the chunk that holds key Sk - 1: element by element
      for (int u = 0; u < LF_BC_BM / 4; ++u) {
        const int q = min(q0 + 4 * u + r4, qlast);
        for (int e = 0; j + e <= klast; ++e) {
          const unsigned b16 = bits(q, j + e);
          dead = dead && lf_bias_masked(b16);
          zero = zero && is_zero(b16);
        }
      }
    }
  }
  const bool all_dead = __builtin_amdgcn_ballot_w64(dead) == ~0ull;
  const bool all_zero = __builtin_amdgcn_ballot_w64(zero) == ~0ull;
  if (lane == 0) cls[kt] = all_dead ? 0 : (all_zero ? 1 : 2);
}
