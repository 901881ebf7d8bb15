/*
 * lf_client.c — a C host that drives the attention kernels through the C ABI alone
 * (include/lf_shim.h + include/lf_attn_params.h): no Python, no torch.
 *
 *   lf_client <kernel source dir> [prefill|prefill_swp|decode]
 *
 * It compiles lf_attn_prefill.hip or lf_attn_prefill_swp.hip (causal, bf16, D = 128) or lf_attn_decode.hip
 * (paged GQA, bf16, D = 128, pages of 16 tokens) with lf_compile, loads and
 * launches it with lf_module_load / lf_get_function / lf_launch on device buffers
 * of its own, and checks the result against double-precision loops over the same
 * bf16-rounded inputs.  Exit status 0 and a line "OK ..." on success.
 *
 * Test infrastructure: the loops below are a checker, not a CPU path of the library.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "lf_attn_params.h"
#include "lf_shim.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { \
  fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); return 2; } } while (0)
#define CHECK_LF(x) do { int e_ = (x); if (e_ != 0) { \
  fprintf(stderr, "%s -> %d: %s\n", #x, e_, lf_last_error()); return 3; } } while (0)

static uint16_t to_bf16(float f) {           /* round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t rng_state = 12345u;
static float rnd(void) {                      /* roughly N(0, 1): sum of 4 uniforms */
  float s = 0.0f;
  for (int i = 0; i < 4; ++i) {
    rng_state = rng_state * 1664525u + 1013904223u;
    s += (float)(rng_state >> 8) / 16777216.0f - 0.5f;
  }
  return s * 1.7320508f;
}
static void fill(uint16_t* p, size_t n) { for (size_t i = 0; i < n; ++i) p[i] = to_bf16(rnd()); }

static char* read_file(const char* dir, const char* name, size_t* len) {
  char path[4096];
  snprintf(path, sizeof path, "%s/%s", dir, name);
  FILE* f = fopen(path, "rb");
  if (!f) { perror(path); return NULL; }
  fseek(f, 0, SEEK_END);
  long n = ftell(f);
  fseek(f, 0, SEEK_SET);
  char* buf = (char*)malloc((size_t)n + 1);
  if (fread(buf, 1, (size_t)n, f) != (size_t)n) { fclose(f); free(buf); return NULL; }
  fclose(f);
  buf[n] = 0;
  *len = (size_t)n;
  return buf;
}

/* common header (+ the prefill building blocks) + kernel file = one translation unit */
static char* kernel_source(const char* dir, const char* file) {
  const char* parts[3] = {"lf_common.hip.h", strstr(file, "prefill") ? "lf_prefill_blocks.hip.h" : NULL, file};
  char* s = (char*)malloc(1);
  size_t total = 0;
  s[0] = 0;
  for (int i = 0; i < 3; ++i) {
    if (!parts[i]) continue;
    size_t n;
    char* t = read_file(dir, parts[i], &n);
    if (!t) { free(s); return NULL; }
    s = (char*)realloc(s, total + n + 2);
    memcpy(s + total, t, n);
    s[total + n] = '\n';
    s[total + n + 1] = 0;
    total += n + 1;
    free(t);
  }
  return s;
}

static int load_kernel(const char* dir, const char* file, const char* const* opts, int nopts,
                       const char* symbol, void** fn) {
  char* src = kernel_source(dir, file);
  if (!src) return 4;
  void* code = NULL;
  size_t len = 0;
  char log[4096];
  log[0] = 0;
  int rc = lf_compile(src, file, opts, nopts, "gfx950", &code, &len, log, sizeof log);
  free(src);
  if (rc != 0) { fprintf(stderr, "lf_compile -> %d: %s\n%s\n", rc, lf_last_error(), log); return 3; }
  void* mod = NULL;
  CHECK_LF(lf_module_load(code, len, &mod));
  lf_free_code(code);
  CHECK_LF(lf_get_function(mod, symbol, fn));
  return 0;
}

static const char* kCommon[] = {"-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                                "-DLF_DTYPE=0", "-DLF_HEAD_DIM=128", "-DLF_SOFTCAP=0", "-DLF_TABLE_I64=0"};
#define NCOMMON ((int)(sizeof kCommon / sizeof kCommon[0]))

static int run_prefill(const char* dir, const char* file, const char* symbol) {
  enum { B = 2, H = 3, S = 200, D = 128 };
  const size_t n = (size_t)B * H * S * D;
  uint16_t *q = malloc(2 * n), *k = malloc(2 * n), *v = malloc(2 * n), *o = malloc(2 * n);
  fill(q, n); fill(k, n); fill(v, n);
  void *dq, *dk, *dv, *dout;
  CHECK_HIP(hipMalloc(&dq, 2 * n)); CHECK_HIP(hipMalloc(&dk, 2 * n));
  CHECK_HIP(hipMalloc(&dv, 2 * n)); CHECK_HIP(hipMalloc(&dout, 2 * n));
  CHECK_HIP(hipMemcpy(dq, q, 2 * n, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dk, k, 2 * n, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dv, v, 2 * n, hipMemcpyHostToDevice));

  const char* opts[NCOMMON + 3];
  memcpy(opts, kCommon, sizeof kCommon);
  opts[NCOMMON] = "-DLF_MASK=1"; opts[NCOMMON + 1] = "-DLF_PAGED=0"; opts[NCOMMON + 2] = "-DLF_PAGE_SIZE=1";
  void* fn = NULL;
  int rc = load_kernel(dir, file, opts, NCOMMON + 3, symbol, &fn);
  if (rc) return rc;

  LfAttnParamsHost p;
  memset(&p, 0, sizeof p);
  p.q = dq; p.k = dk; p.v = dv; p.o = dout;
  p.q_sb = p.k_sb = p.v_sb = p.o_sb = (int64_t)H * S * D;
  p.q_sh = p.k_sh = p.v_sh = p.o_sh = (int64_t)S * D;
  p.q_ss = p.k_ss = p.v_ss = p.o_ss = D;
  p.B = B; p.Hq = H; p.Hkv = H; p.Sq = S; p.Sk = S;
  p.nsplit = 1; p.rows = 1; p.k2_group = 1;
  p.scale = 1.0f / sqrtf((float)D);
  /* lf_attn_prefill: 8 XCD classes x (batch*head pairs per class, in groups of 4) x pairs of
     128-row q tiles; lf_attn_prefill_swp: groups of 8, one q tile per workgroup */
  const unsigned per_xcd = (B * H + 7) / 8, nqt = (S + 127) / 128;
  const unsigned grid = strcmp(symbol, "lf_attn_prefill_swp") == 0 ? 8 * ((per_xcd + 7) / 8 * 8) * nqt
                                                                     : 8 * ((per_xcd + 3) / 4 * 4) * ((nqt + 1) / 2);
  void* args[1] = {&p};
  CHECK_LF(lf_launch(fn, grid, 1, 1, 256, 1, 1, 0, NULL, args));
  CHECK_HIP(hipDeviceSynchronize());
  CHECK_HIP(hipMemcpy(o, dout, 2 * n, hipMemcpyDeviceToHost));

  double worst = 0.0;
  double* w = malloc(sizeof(double) * S);
  for (int b = 0; b < B; ++b) for (int h = 0; h < H; ++h) for (int i = 0; i < S; ++i) {
    const uint16_t* qi = q + (((size_t)b * H + h) * S + i) * D;
    double mx = -1e300, tot = 0.0;
    for (int j = 0; j <= i; ++j) {
      const uint16_t* kj = k + (((size_t)b * H + h) * S + j) * D;
      double s = 0.0;
      for (int d = 0; d < D; ++d) s += (double)from_bf16(qi[d]) * from_bf16(kj[d]);
      w[j] = s * p.scale;
      if (w[j] > mx) mx = w[j];
    }
    for (int j = 0; j <= i; ++j) { w[j] = exp(w[j] - mx); tot += w[j]; }
    for (int d = 0; d < D; ++d) {
      double acc = 0.0;
      for (int j = 0; j <= i; ++j) acc += w[j] * from_bf16(v[(((size_t)b * H + h) * S + j) * D + d]);
      const double err = fabs(acc / tot - from_bf16(o[(((size_t)b * H + h) * S + i) * D + d]));
      if (!(err <= worst)) worst = err;      /* NaN-proof */
    }
  }
  printf("%s causal bf16 B%d H%d S%d D%d through the C ABI: max abs err %.3g\n", symbol, B, H, S, D, worst);
  return worst <= 2e-2 ? 0 : 1;
}

static int run_decode(const char* dir) {
  /* paged GQA decode: pools [N, 16, Hkv, D], table [B, S/16], 4 query heads per kv head */
  enum { B = 3, HKV = 2, G = 4, S = 320, D = 128, P = 16, PAGES = S / P, N = B * PAGES };
  const size_t nq = (size_t)B * HKV * G * D, npool = (size_t)N * P * HKV * D;
  uint16_t *q = malloc(2 * nq), *kp = malloc(2 * npool), *vp = malloc(2 * npool), *o = malloc(2 * nq);
  int32_t* table = malloc(sizeof(int32_t) * N);
  fill(q, nq); fill(kp, npool); fill(vp, npool);
  for (int i = 0; i < N; ++i) table[i] = (i * 7 + 3) % N;          /* a permutation: 7 and N = 60 are coprime */
  void *dq, *dk, *dv, *dout, *dt;
  CHECK_HIP(hipMalloc(&dq, 2 * nq)); CHECK_HIP(hipMalloc(&dout, 2 * nq));
  CHECK_HIP(hipMalloc(&dk, 2 * npool)); CHECK_HIP(hipMalloc(&dv, 2 * npool));
  CHECK_HIP(hipMalloc(&dt, sizeof(int32_t) * N));
  CHECK_HIP(hipMemcpy(dq, q, 2 * nq, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dk, kp, 2 * npool, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dv, vp, 2 * npool, hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(dt, table, sizeof(int32_t) * N, hipMemcpyHostToDevice));

  const char* opts[NCOMMON + 5];
  memcpy(opts, kCommon, sizeof kCommon);
  opts[NCOMMON] = "-DLF_MASK=0"; opts[NCOMMON + 1] = "-DLF_PAGED=3"; opts[NCOMMON + 2] = "-DLF_PAGE_SIZE=16";
  opts[NCOMMON + 3] = "-DLF_DW=4"; opts[NCOMMON + 4] = "-DLF_HEADWAVE=0";
  void* fn = NULL;
  int rc = load_kernel(dir, "lf_attn_decode.hip", opts, NCOMMON + 5, "lf_attn_decode", &fn);
  if (rc) return rc;

  LfAttnParamsHost p;
  memset(&p, 0, sizeof p);
  p.q = dq; p.k = dk; p.v = dv; p.o = dout; p.k_table = dt; p.v_table = dt;
  /* one unit = (batch, kv head) with its G query heads as rows */
  p.q_sb = p.o_sb = (int64_t)HKV * G * D; p.q_sh = p.o_sh = (int64_t)G * D; p.q_ss = p.o_ss = D;
  p.k_sb = p.v_sb = (int64_t)P * HKV * D;      /* page stride */
  p.k_ss = p.v_ss = (int64_t)HKV * D;          /* token stride inside a page */
  p.k_sh = p.v_sh = D;
  p.B = B; p.Hq = HKV * G; p.Hkv = HKV; p.Sq = 1; p.Sk = S;
  p.kt_stride = p.vt_stride = PAGES;
  p.nsplit = 1; p.rows = G; p.split_len = S; p.k2_group = 1;
  p.scale = 1.0f / sqrtf((float)D);
  void* args[1] = {&p};
  CHECK_LF(lf_launch(fn, B * HKV, 1, 1, 256, 1, 1, 0, NULL, args));
  CHECK_HIP(hipDeviceSynchronize());
  CHECK_HIP(hipMemcpy(o, dout, 2 * nq, hipMemcpyDeviceToHost));

  double worst = 0.0, w[S];
  for (int b = 0; b < B; ++b) for (int h = 0; h < HKV * G; ++h) {
    const int hk = h / G;
    const uint16_t* qi = q + ((size_t)b * HKV * G + h) * D;
    double mx = -1e300, tot = 0.0;
    for (int j = 0; j < S; ++j) {
      const size_t row = (((size_t)table[b * PAGES + j / P] * P + j % P) * HKV + hk) * D;
      double s = 0.0;
      for (int d = 0; d < D; ++d) s += (double)from_bf16(qi[d]) * from_bf16(kp[row + d]);
      w[j] = s * p.scale;
      if (w[j] > mx) mx = w[j];
    }
    for (int j = 0; j < S; ++j) { w[j] = exp(w[j] - mx); tot += w[j]; }
    for (int d = 0; d < D; ++d) {
      double acc = 0.0;
      for (int j = 0; j < S; ++j)
        acc += w[j] * from_bf16(vp[(((size_t)table[b * PAGES + j / P] * P + j % P) * HKV + hk) * D + d]);
      const double err = fabs(acc / tot - from_bf16(o[((size_t)b * HKV * G + h) * D + d]));
      if (!(err <= worst)) worst = err;
    }
  }
  printf("decode paged GQA bf16 B%d Hq%d Hkv%d S%d D%d page %d through the C ABI: max abs err %.3g\n",
         B, HKV * G, HKV, S, D, P, worst);
  return worst <= 2e-2 ? 0 : 1;
}

int main(int argc, char** argv) {
  if (argc < 2) { fprintf(stderr, "usage: %s <kernel source dir> [prefill|prefill_swp|decode]\n", argv[0]); return 64; }
  if (lf_abi_version() != 2) { fprintf(stderr, "unexpected ABI version %d\n", lf_abi_version()); return 5; }
  char arch[64];
  int cus = 0, lds = 0;
  CHECK_LF(lf_device_info(0, arch, sizeof arch, &cus, &lds));
  printf("device 0: %s, %d CUs, %d bytes of LDS per workgroup\n", arch, cus, lds);
  int rc = 0;
  if (argc < 3 || !strcmp(argv[2], "prefill")) rc |= run_prefill(argv[1], "lf_attn_prefill.hip", "lf_attn_prefill");
  if (argc < 3 || !strcmp(argv[2], "prefill_swp")) rc |= run_prefill(argv[1], "lf_attn_prefill_swp.hip", "lf_attn_prefill_swp");
  if (argc < 3 || !strcmp(argv[2], "decode")) rc |= run_decode(argv[1]);
  if (rc == 0) printf("OK\n");
  return rc;
}
