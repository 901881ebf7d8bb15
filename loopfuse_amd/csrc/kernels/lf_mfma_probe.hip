// lf_mfma_probe.hip — what the matrix cores of this GPU sustain on given operand DATA.
//
// One launch = `iters` rounds of 32 independent v_mfma_f32_32x32x16_bf16 (KIND 0) or 64
// v_mfma_f32_16x16x32_bf16 (KIND 1) per wave, operands resident in registers, accumulators in
// four / eight independent chains; nothing else in the loop.  The operands come from `data`
// (64 Ki 16-byte pieces), so the same code can be timed on zeros, ones or N(0,1) values: the
// chip lowers its clock with the switching activity of the operands, and the rate this probe
// reaches on the benchmark's own input distribution is the ceiling of any MFMA-bound kernel
// on it.  Thread 0 of each workgroup also reports shader cycles and 100 MHz ticks, which
// gives the average shader clock during the launch.
#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif

struct LfProbeParams {
  float* out;
  const unsigned int* data;
  unsigned long long* clk;   // [gridDim.x][2]: shader cycles, 100 MHz ticks
  int iters;
};

typedef __bf16 lfp_bf16x8 __attribute__((ext_vector_type(8)));
typedef float lfp_f32x16 __attribute__((ext_vector_type(16)));
typedef float lfp_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int lfp_u32x4 __attribute__((ext_vector_type(4)));

#ifndef LF_PROBE_KIND
#define LF_PROBE_KIND 0
#endif

extern "C" __global__ void __launch_bounds__(256, 2) lf_mfma_probe(const LfProbeParams p) {
  const int tid = threadIdx.x;
  lfp_u32x4 q[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
    q[i] = reinterpret_cast<const lfp_u32x4*>(p.data)[(blockIdx.x * 256 + tid + 300 * i) % 65536];
  const unsigned long long t0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  float r = 0.f;
#if LF_PROBE_KIND == 1
  lfp_f32x4 o[8];
#pragma unroll
  for (int k = 0; k < 8; ++k)
#pragma unroll
    for (int i = 0; i < 4; ++i) o[k][i] = 0.f;
  for (int it = 0; it < p.iters; ++it) {
#pragma unroll
    for (int f = 0; f < 64; ++f)
      o[f & 7] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lfp_bf16x8, q[f & 7]),
                                                         __builtin_bit_cast(lfp_bf16x8, q[(f + 3) & 7]), o[f & 7], 0, 0, 0);
  }
#pragma unroll
  for (int k = 0; k < 8; ++k)
#pragma unroll
    for (int i = 0; i < 4; ++i) r += o[k][i];
#else
  lfp_f32x16 o[4];
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[k][i] = 0.f;
  for (int it = 0; it < p.iters; ++it) {
#pragma unroll
    for (int f = 0; f < 32; ++f)
      o[f & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(lfp_bf16x8, q[f & 7]),
                                                         __builtin_bit_cast(lfp_bf16x8, q[(f + 3) & 7]), o[f & 3], 0, 0, 0);
  }
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += o[k][i];
#endif
  const unsigned long long t1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  if (tid == 0) {
    p.clk[2 * blockIdx.x] = t1 - t0;
    p.clk[2 * blockIdx.x + 1] = r1 - r0;
  }
  p.out[blockIdx.x * 256 + tid] = r;
}
