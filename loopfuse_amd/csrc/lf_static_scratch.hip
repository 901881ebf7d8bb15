// lf_static_scratch.hip — the one entry point of liblf_shim.so that needs no caller-side
// scratch allocation: lf_launch_decode_static (declared in include/lf_shim.h).
//
// A split decode step runs two kernels of one code object: lf_attn_decode, which writes one
// partial result (exponent offset, sum, accumulator) per (unit, row, KV split), and
// lf_attn_decode_combine, which merges them into O.  Through lf_launch the caller owns the
// buffer those partials live in.  Here it is a file-scope device array instead, so that callers
// which cannot allocate (a stream under HIP graph capture, a serving loop, a harness that forbids
// hipMalloc) can still run the step.  Each GPU the library runs on holds its own copy of the array
// (LF_STATIC_SCRATCH_BYTES) at its own address until the process ends; the address is looked up
// once per device, with that device current, and only that looked-up pointer is ever used.
//
// Every launch on a GPU shares that GPU's array: two calls that overlap on one GPU (different
// streams) race on it.  Calls on one stream are ordered and safe.  Nothing has to start at zero:
// the streaming kernel writes every partial the combine kernel reads in the same step.
#include <hip/hip_runtime.h>

#include <cstring>
#include <mutex>
#include <string>

#include "lf_attn_params.h"
#include "lf_shim.h"
#include "lf_shim_internal.h"

static __device__ __align__(256) unsigned char scratch[LF_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_mu;
unsigned char* g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each GPU (0 = not looked up yet)

// Device address of this GPU's copy of the array (the array's name is only a host-side handle).
int scratch_for_current_device(unsigned char** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return lf_internal_fail(static_cast<int>(e), std::string("lf_launch_decode_static: hipGetDevice: ") + hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return lf_internal_fail(LF_EINVAL, "lf_launch_decode_static: device index out of range");
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return lf_internal_fail(e != hipSuccess ? static_cast<int>(e) : LF_EINVAL,
                              std::string("lf_launch_decode_static: hipGetSymbolAddress: ") + hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

}  // namespace

extern "C" {

size_t lf_static_scratch_bytes(void) { return LF_STATIC_SCRATCH_BYTES; }

int lf_launch_decode_static(void* fn_decode, void* fn_combine, const void* params, size_t params_bytes,
                            size_t part_acc_bytes, size_t part_ml_bytes,
                            unsigned gx, unsigned gy, unsigned bx,
                            unsigned combine_gx, unsigned combine_bx, void* stream) {
  if (!fn_decode || !fn_combine || !params)
    return lf_internal_fail(LF_EINVAL, "lf_launch_decode_static: null function or parameter block");
  if (params_bytes != sizeof(LfAttnParamsHost))
    return lf_internal_fail(LF_EINVAL, "lf_launch_decode_static: parameter block has the wrong size");
  if (gx == 0 || gy == 0 || bx == 0 || combine_gx == 0 || combine_bx == 0 || bx > 1024 || combine_bx > 1024)
    return lf_internal_fail(LF_EINVAL, "lf_launch_decode_static: bad launch geometry");
  // the two regions, each rounded up to the array's alignment
  const size_t acc = (part_acc_bytes + 255) / 256 * 256;
  const size_t ml = (part_ml_bytes + 255) / 256 * 256;
  if (part_acc_bytes == 0 || part_ml_bytes == 0 || acc > LF_STATIC_SCRATCH_BYTES || ml > LF_STATIC_SCRATCH_BYTES - acc)
    return lf_internal_fail(LF_ENOSPC, "lf_launch_decode_static: the split-K partials need " +
                                           std::to_string(acc + ml) + " bytes, the static scratch holds " +
                                           std::to_string(static_cast<size_t>(LF_STATIC_SCRATCH_BYTES)) +
                                           " (fewer splits, or lf_launch with a caller-owned buffer)");
  unsigned char* base = nullptr;
  if (int rc = scratch_for_current_device(&base)) return rc;

  LfAttnParamsHost p;
  std::memcpy(&p, params, sizeof p);
  p.part_acc = reinterpret_cast<float*>(base);
  p.part_ml = reinterpret_cast<float*>(base + acc);
  void* args[1] = {&p};
  hipError_t e = hipModuleLaunchKernel(static_cast<hipFunction_t>(fn_decode), gx, gy, 1, bx, 1, 1, 0,
                                       static_cast<hipStream_t>(stream), args, nullptr);
  if (e != hipSuccess)
    return lf_internal_fail(static_cast<int>(e), std::string("lf_launch_decode_static: decode launch: ") + hipGetErrorString(e));
  e = hipModuleLaunchKernel(static_cast<hipFunction_t>(fn_combine), combine_gx, 1, 1, combine_bx, 1, 1, 0,
                            static_cast<hipStream_t>(stream), args, nullptr);
  if (e != hipSuccess)
    return lf_internal_fail(static_cast<int>(e), std::string("lf_launch_decode_static: combine launch: ") + hipGetErrorString(e));
  return 0;
}

}  // extern "C"
