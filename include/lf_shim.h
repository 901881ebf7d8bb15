/*
 * lf_shim.h — C ABI of the loopfuse MI355X runtime shim (liblf_shim.so).
 *
 * The reference has no FFI of its own: its lowering writes Triton source to a
 * temporary .py file, imports it and calls the generated launch function
 * (reference loopfuse/torch_backend/interface.py:624-644, loopfuse/codegen.py:
 * 215-298).  This library is the seam that replaces that step: the Python
 * lowering hands it HIP source plus -D specialisation options, gets a gfx950
 * code object back (hipRTC), loads it and launches kernels on a caller-supplied
 * HIP stream.  Plain pointers and sizes only; no torch types.
 *
 * Conventions
 *   - every function returning int returns 0 on success, otherwise the
 *     hip/hiprtc error code (or a negative LF_E* code); a human-readable
 *     message for the calling thread is available from lf_last_error().
 *   - the shim never allocates device memory; every device buffer (inputs,
 *     outputs, split-K scratch) belongs to the caller.  lf_launch_decode_static
 *     is the one exception to the last item: its split-K scratch is a static
 *     device array inside the library.
 *   - all entry points are re-entrant; the only shared state is an
 *     internally locked table of loaded modules.
 */
#ifndef LF_SHIM_H
#define LF_SHIM_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LF_EINVAL (-1)   /* bad argument */
#define LF_EIO    (-2)   /* cache file could not be read/written */
#define LF_ENOSYM (-3)   /* kernel symbol not found in module */
#define LF_ENOSPC (-4)   /* request larger than the library's static scratch */

/* Size of the static device array behind lf_launch_decode_static (one copy per GPU the
 * library runs on, held until the process ends). */
#define LF_STATIC_SCRATCH_BYTES (8u << 20)

/* ABI version of this header; bumped on any signature change. */
int lf_abi_version(void);

/* Message describing the last failure on the calling thread ("" if none). */
const char* lf_last_error(void);

/*
 * Compile HIP source to a code object for `arch` (e.g. "gfx950") with hipRTC.
 * Replaces: emission + import of the generated Triton module and Triton's JIT
 * (reference interface.py:624-638, codegen.py:163-168, 386-404).
 *   src, name      : NUL-terminated source text and a file name for diagnostics
 *   opts, nopts    : extra compiler options ("-DLF_HEAD_DIM=128", ...)
 *   arch           : offload architecture; NULL/"" = architecture of device 0
 *   code, code_len : out, malloc'ed code object; release with lf_free_code
 *   log, log_cap   : optional buffer receiving the compiler log (NUL-terminated)
 * Works without a GPU when `arch` is given.
 */
int lf_compile(const char* src, const char* name,
               const char* const* opts, int nopts, const char* arch,
               void** code, size_t* code_len, char* log, size_t log_cap);

/*
 * As lf_compile, but looks the result up in / stores it into `cache_dir`,
 * keyed by a 64-bit FNV-1a hash of source, options and arch.  `hit`
 * (optional) is set to 1 when the code object came from the cache.
 * Replaces triton.autotune/JIT's on-disk cache (reference codegen.py:386-393).
 */
int lf_compile_cached(const char* src, const char* name,
                      const char* const* opts, int nopts, const char* arch,
                      const char* cache_dir,
                      void** code, size_t* code_len, int* hit,
                      char* log, size_t log_cap);

void lf_free_code(void* code);

/* Load a code object on the current device / look a kernel up in it.
 * Replaces importlib loading of the generated module and getattr(launch_name)
 * (reference interface.py:626-638). */
int lf_module_load(const void* code, size_t len, void** mod);
int lf_get_function(void* mod, const char* sym, void** fn);
int lf_module_unload(void* mod);

/*
 * Launch `fn` asynchronously on `stream` (a hipStream_t; NULL = default
 * stream).  `args` is an array with one pointer per kernel parameter.
 * Replaces the generated launch function's `kernel_0[grid](...)` call
 * (reference codegen.py:288-298).  No host synchronisation.
 */
int lf_launch(void* fn, unsigned gx, unsigned gy, unsigned gz,
              unsigned bx, unsigned by, unsigned bz,
              unsigned lds_bytes, void* stream, void** args);

/*
 * No counterpart in the reference.  For callers that cannot allocate device memory
 * (a stream under HIP graph capture, a tight serving loop, a harness that forbids
 * hipMalloc): one split decode step -- `fn_decode` (lf_attn_decode) on a (gx, gy)
 * grid of bx threads, then `fn_combine` (lf_attn_decode_combine) on combine_gx
 * blocks of combine_bx threads, both from one code object and both taking
 * `params` (an LfAttnParamsHost, include/lf_attn_params.h) by value -- with the
 * split-K partials in a static device array of LF_STATIC_SCRATCH_BYTES instead of a
 * caller-owned buffer: the part_acc / part_ml fields of `params` are ignored and
 * replaced.  part_acc_bytes / part_ml_bytes say how much the step needs
 * (units * nsplit * rows * D * 4 and units * nsplit * rows * 2 * 4); more than the
 * array holds is refused with LF_ENOSPC.  Allocates nothing and frees nothing.
 * Every call on a GPU shares that GPU's array: calls on one stream are ordered,
 * calls that overlap on one GPU (different streams) race.  The array keeps the last
 * call's partials; nothing in it has to start at zero.
 */
int lf_launch_decode_static(void* fn_decode, void* fn_combine,
                            const void* params, size_t params_bytes,
                            size_t part_acc_bytes, size_t part_ml_bytes,
                            unsigned gx, unsigned gy, unsigned bx,
                            unsigned combine_gx, unsigned combine_bx, void* stream);

/* LF_STATIC_SCRATCH_BYTES as the built library has it. */
size_t lf_static_scratch_bytes(void);

/* Architecture name, compute-unit count and LDS bytes per workgroup of a
 * device.  Fails (non-zero) when there is no usable GPU. */
int lf_device_info(int dev, char* arch, size_t cap, int* cus, int* lds_bytes);

/* Number of visible HIP devices (0 when none / no driver). */
int lf_device_count(void);

#ifdef __cplusplus
}
#endif
#endif /* LF_SHIM_H */
