// lf_prefill_blocks.hip.h — building blocks shared by the prefill kernels
// (lf_attn_prefill.hip, lf_attn_prefill_swp.hip): K/V tile geometry in LDS, the XOR
// swizzles, the MFMA fragment readers, direct-to-LDS staging and the mask predicate.
//
// Tile layout.  A K or V tile holds LF_BN rows of LF_D elements, row-major and unpadded;
// the 16-byte chunks of a row are permuted by an XOR with the row index so that both
// read patterns below touch every LDS bank once.  Fragment orders (32x32x16 MFMA, lane =
// (l32 = lane % 32, g = lane / 32)):
//   K fragment f = ks * LF_NKB + kb : A operand of S^T = K Q^T, row = key 32*kb + l32,
//                                     k = d 16*ks + 8*g .. +7             (one ds_read_b128)
//   V fragment f = kk * LF_NDB + db : A operand of O^T += V^T P^T, row = d 32*db + l32,
//                                     k-slot s = key 16*kk + 8*(s/4) + 4*g + s%4, the order
//                                     the accumulator of S^T holds P in   (two ds_read_b64_tr_b16)
#ifndef LF_PREFILL_BLOCKS_HIP_H
#define LF_PREFILL_BLOCKS_HIP_H

#ifndef LF_BN
#define LF_BN 64                             /* keys per LDS tile             */
#endif
#define LF_D LF_HEAD_DIM
#define LF_CPR (LF_D / 8)                    /* 16-byte chunks per K/V row    */
#define LF_RPS (256 / (LF_D * 2))            /* rows per 256-byte bank span   */
#define LF_NKB (LF_BN / 32)                  /* 32-row blocks of S^T per tile */
#define LF_NKS (LF_D / 16)                   /* k-steps of the QK^T product   */
#define LF_NDB (LF_D / 32)                   /* 32-row blocks of O^T          */
#define LF_NKK (LF_BN / 16)                  /* k-steps of the PV product     */

// Physical 16-byte chunk of logical chunk `ch` in row `row` of the K tile: rows that a
// ds_read_b128 touches together (16 consecutive rows, same logical chunk) land in 16
// different chunks, i.e. on all 64 banks.
__device__ __forceinline__ int lf_k_phys(int row, int ch) {
  return ch ^ ((row / LF_RPS) & (LF_CPR - 1));
}
// Same for the V tile, where a transposed read touches 4 consecutive rows x 64 contiguous
// bytes per 32 lanes: permute the 64-byte groups by the row.
__device__ __forceinline__ int lf_v_phys(int row, int ch) {
  return ch ^ (4 * ((row / LF_RPS) & (LF_CPR / 4 - 1)));
}

__device__ __forceinline__ lf_u32x4 lf_read_k_frag(const lf_elem* kbuf, int l32, int g, int f) {
  const int ks = f / LF_NKB, kb = f % LF_NKB;
  const int row = 32 * kb + l32;
  return *reinterpret_cast<const lf_u32x4*>(&kbuf[row * LF_D + 8 * lf_k_phys(row, 2 * ks + g)]);
}

// 16-lane group (2g + dh) asks for rows r0..r0+3, columns 32db+16dh..+15: lane j of the
// group supplies the 8-byte piece (row r0 + j/4, cols +4*(j%4)) and receives column j of
// the 4 rows.
__device__ __forceinline__ lf_elem8 lf_read_v_frag_tr(const lf_elem* vbuf, int lane, int g, int f) {
  const int kk = f / LF_NDB, db = f % LF_NDB;
  const int j16 = lane & 15;
  const int dh = (lane >> 4) & 1;
  const int col = 32 * db + 16 * dh + 4 * (j16 & 3);
  lf_elem8 a;
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
  return a;
}

// One wave-level direct-to-LDS load: 64 lanes x 16 B land at lds_row0 + 16 * lane; lane
// offsets `voff` are bytes inside the buffer resource `rs`, a range-checked offset beyond
// the resource delivers zeros.  The load is not tracked by the compiler's wait counters:
// callers wait with s_waitcnt vmcnt themselves.  m0 is declared as an output so that the
// compiler knows the statement overwrites it.
__device__ __forceinline__ void lf_dma_to_lds(const lf_u32x4& rs, unsigned voff, const lf_elem* lds_row0) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane(
      (unsigned)(size_t)(__attribute__((address_space(3))) const void*)lds_row0);
  unsigned m0_written;
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %3, 0 offen lds"
               : "={m0}"(m0_written) : "s"(m0v), "v"(voff), "s"(rs) : "memory");
}

// The same with the destination given as an LDS byte address (a wave-uniform integer, see lf_lds_addr): a
// pointer that went through run-time arithmetic comes back from its generic form with a null test per load.
__device__ __forceinline__ void lf_dma_to_lds_at(const lf_u32x4& rs, unsigned voff, unsigned lds_addr) {
  unsigned m0_written;
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %3, 0 offen lds"
               : "={m0}"(m0_written) : "s"(lds_addr), "v"(voff), "s"(rs) : "memory");
}
// LDS byte address of a __shared__ object (folds to a constant for the object itself).
#define lf_lds_addr(obj) ((unsigned)(size_t)(__attribute__((address_space(3))) const void*)(obj))

// Buffer resource over `bytes` bytes from `base` (raw buffer, 32-bit offsets, range checked).
__device__ __forceinline__ lf_u32x4 lf_make_buffer(const void* base, unsigned bytes) {
  const unsigned long long a = (unsigned long long)base;
  lf_u32x4 rs;
  rs[0] = __builtin_amdgcn_readfirstlane((unsigned)a);
  rs[1] = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32) & 0xffffu);
  rs[2] = __builtin_amdgcn_readfirstlane(bytes);
  rs[3] = 0x00020000u;
  return rs;
}

// Is score (query row q, key j) kept?  Top-left aligned masks of the reference
// (loopfuse/torch_backend/ops.py:675-751) plus the bound of the key sequence.
__device__ __forceinline__ bool lf_mask_keep(int q, int j, int Sk, int window) {
  bool ok = j < Sk;
#if LF_MASK >= 1
  ok = ok && (j <= q);
#endif
#if LF_MASK == 2
  ok = ok && (q - j < window);
#endif
  (void)window;
  return ok;
}

#endif  // LF_PREFILL_BLOCKS_HIP_H
