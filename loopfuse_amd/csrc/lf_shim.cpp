// lf_shim.cpp — C-ABI runtime shim: hipRTC compile (+ on-disk cache), module
// load, kernel launch.  Declarations and the reference seam each entry point
// replaces are in include/lf_shim.h.
//
// Host-only C++; links libhiprtc and libamdhip64.  When loaded into a process
// that already holds PyTorch-ROCm, the dynamic linker resolves both by soname to
// the copies torch loaded, so streams and device pointers are shared with torch.
#include "lf_shim.h"
#include "lf_shim_internal.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <cerrno>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_set>
#include <vector>

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

namespace {

thread_local std::string g_err;

int fail(int code, const std::string& msg) {
  g_err = msg;
  return code;
}

int fail_hip(hipError_t e, const char* what) {
  g_err = std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")";
  return static_cast<int>(e);
}

int fail_rtc(hiprtcResult r, const char* what) {
  g_err = std::string(what) + ": " + hiprtcGetErrorString(r);
  return static_cast<int>(r);
}

// Loaded modules, so lf_get_function / lf_module_unload can reject stale handles.
std::mutex g_mod_mu;
std::unordered_set<void*> g_mods;

uint64_t fnv1a(uint64_t h, const void* p, size_t n) {
  const unsigned char* b = static_cast<const unsigned char*>(p);
  for (size_t i = 0; i < n; ++i) {
    h ^= b[i];
    h *= 1099511628211ull;
  }
  return h;
}

uint64_t hash_request(const char* src, const char* const* opts, int nopts, const char* arch) {
  uint64_t h = 1469598103934665603ull;
  h = fnv1a(h, src, std::strlen(src));
  for (int i = 0; i < nopts; ++i) {
    h = fnv1a(h, "\x1f", 1);
    h = fnv1a(h, opts[i], std::strlen(opts[i]));
  }
  h = fnv1a(h, "\x1e", 1);
  h = fnv1a(h, arch, std::strlen(arch));
  return h;
}

void copy_log(const std::string& s, char* log, size_t cap) {
  if (!log || cap == 0) return;
  size_t n = s.size() < cap - 1 ? s.size() : cap - 1;
  std::memcpy(log, s.data(), n);
  log[n] = '\0';
}

int resolve_arch(const char* arch, std::string* out) {
  if (arch && arch[0]) {
    *out = arch;
    return 0;
  }
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, 0);
  if (e != hipSuccess) return fail_hip(e, "lf_compile: no arch given and no device");
  std::string a = prop.gcnArchName;  // "gfx950:sramecc+:xnack-"
  size_t c = a.find(':');
  *out = c == std::string::npos ? a : a.substr(0, c);
  return 0;
}

}  // namespace

int lf_internal_fail(int code, const std::string& msg) { return fail(code, msg); }

extern "C" {

int lf_abi_version(void) { return 2; }

const char* lf_last_error(void) { return g_err.c_str(); }

int lf_compile(const char* src, const char* name, const char* const* opts, int nopts,
               const char* arch, void** code, size_t* code_len, char* log, size_t log_cap) {
  if (!src || !code || !code_len || nopts < 0 || (nopts > 0 && !opts))
    return fail(LF_EINVAL, "lf_compile: bad argument");
  *code = nullptr;
  *code_len = 0;
  if (log && log_cap) log[0] = '\0';
  std::string a;
  if (int rc = resolve_arch(arch, &a)) return rc;

  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, src, name ? name : "lf_kernel.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail_rtc(r, "hiprtcCreateProgram");

  std::string archopt = "--offload-arch=" + a;
  std::vector<const char*> all;
  all.push_back(archopt.c_str());
  for (int i = 0; i < nopts; ++i) all.push_back(opts[i]);
  r = hiprtcCompileProgram(prog, static_cast<int>(all.size()), all.data());

  size_t lsz = 0;
  std::string clog;
  if (hiprtcGetProgramLogSize(prog, &lsz) == HIPRTC_SUCCESS && lsz > 1) {
    clog.resize(lsz);
    hiprtcGetProgramLog(prog, &clog[0]);
    while (!clog.empty() && clog.back() == '\0') clog.pop_back();
  }
  copy_log(clog, log, log_cap);
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    fail_rtc(r, "hiprtcCompileProgram");
    if (!clog.empty()) g_err += "\n" + clog;
    return static_cast<int>(r);
  }
  size_t csz = 0;
  r = hiprtcGetCodeSize(prog, &csz);
  if (r != HIPRTC_SUCCESS || csz == 0) {
    hiprtcDestroyProgram(&prog);
    return fail_rtc(r, "hiprtcGetCodeSize");
  }
  void* buf = std::malloc(csz);
  if (!buf) {
    hiprtcDestroyProgram(&prog);
    return fail(LF_EINVAL, "lf_compile: out of host memory");
  }
  r = hiprtcGetCode(prog, static_cast<char*>(buf));
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    std::free(buf);
    return fail_rtc(r, "hiprtcGetCode");
  }
  *code = buf;
  *code_len = csz;
  return 0;
}

int lf_compile_cached(const char* src, const char* name, const char* const* opts, int nopts,
                      const char* arch, const char* cache_dir, void** code, size_t* code_len,
                      int* hit, char* log, size_t log_cap) {
  if (hit) *hit = 0;
  if (!cache_dir || !cache_dir[0])
    return lf_compile(src, name, opts, nopts, arch, code, code_len, log, log_cap);
  if (!src || !code || !code_len || nopts < 0 || (nopts > 0 && !opts))
    return fail(LF_EINVAL, "lf_compile_cached: bad argument");
  std::string a;
  if (int rc = resolve_arch(arch, &a)) return rc;

  char hex[32];
  std::snprintf(hex, sizeof hex, "%016llx",
                static_cast<unsigned long long>(hash_request(src, opts, nopts, a.c_str())));
  std::string base = name && name[0] ? name : "lf_kernel";
  for (char& c : base)
    if (c == '/' || c == ' ') c = '_';
  std::string path = std::string(cache_dir) + "/" + base + "-" + a + "-" + hex + ".hsaco";

  if (FILE* f = std::fopen(path.c_str(), "rb")) {
    std::fseek(f, 0, SEEK_END);
    long n = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    if (n > 0) {
      void* buf = std::malloc(static_cast<size_t>(n));
      if (buf && std::fread(buf, 1, static_cast<size_t>(n), f) == static_cast<size_t>(n)) {
        std::fclose(f);
        // a hit refreshes the entry's modification time, so that whoever prunes the directory can
        // tell the entries still asked for from superseded ones (failure, e.g. a read-only cache, is fine)
        ::utimensat(AT_FDCWD, path.c_str(), nullptr, 0);
        *code = buf;
        *code_len = static_cast<size_t>(n);
        if (hit) *hit = 1;
        if (log && log_cap) log[0] = '\0';
        return 0;
      }
      std::free(buf);
    }
    std::fclose(f);
  }

  int rc = lf_compile(src, name, opts, nopts, a.c_str(), code, code_len, log, log_cap);
  if (rc) return rc;

  // Store atomically (write to a temporary, then rename); a failed store is not
  // an error for the caller, the compiled code is still returned.
  ::mkdir(cache_dir, 0777);
  std::string tmp = path + ".tmp" + std::to_string(static_cast<long>(::getpid()));
  if (FILE* f = std::fopen(tmp.c_str(), "wb")) {
    bool ok = std::fwrite(*code, 1, *code_len, f) == *code_len;
    ok = (std::fclose(f) == 0) && ok;
    if (!ok || std::rename(tmp.c_str(), path.c_str()) != 0) std::remove(tmp.c_str());
  }
  return 0;
}

void lf_free_code(void* code) { std::free(code); }

int lf_module_load(const void* code, size_t len, void** mod) {
  if (!code || len == 0 || !mod) return fail(LF_EINVAL, "lf_module_load: bad argument");
  *mod = nullptr;
  hipModule_t m;
  hipError_t e = hipModuleLoadData(&m, code);
  if (e != hipSuccess) return fail_hip(e, "hipModuleLoadData");
  {
    std::lock_guard<std::mutex> g(g_mod_mu);
    g_mods.insert(m);
  }
  *mod = m;
  return 0;
}

int lf_get_function(void* mod, const char* sym, void** fn) {
  if (!mod || !sym || !fn) return fail(LF_EINVAL, "lf_get_function: bad argument");
  *fn = nullptr;
  {
    std::lock_guard<std::mutex> g(g_mod_mu);
    if (!g_mods.count(mod)) return fail(LF_EINVAL, "lf_get_function: unknown module handle");
  }
  hipFunction_t f;
  hipError_t e = hipModuleGetFunction(&f, static_cast<hipModule_t>(mod), sym);
  if (e != hipSuccess) {
    fail_hip(e, "hipModuleGetFunction");
    g_err += std::string(" [") + sym + "]";
    return e == hipErrorNotFound ? LF_ENOSYM : static_cast<int>(e);
  }
  *fn = f;
  return 0;
}

int lf_module_unload(void* mod) {
  if (!mod) return fail(LF_EINVAL, "lf_module_unload: bad argument");
  {
    std::lock_guard<std::mutex> g(g_mod_mu);
    if (!g_mods.erase(mod)) return fail(LF_EINVAL, "lf_module_unload: unknown module handle");
  }
  hipError_t e = hipModuleUnload(static_cast<hipModule_t>(mod));
  if (e != hipSuccess) return fail_hip(e, "hipModuleUnload");
  return 0;
}

int lf_launch(void* fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
              unsigned bz, unsigned lds_bytes, void* stream, void** args) {
  if (!fn) return fail(LF_EINVAL, "lf_launch: null function");
  if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0)
    return fail(LF_EINVAL, "lf_launch: empty grid or block");
  if (static_cast<unsigned long long>(bx) * by * bz > 1024ull)
    return fail(LF_EINVAL, "lf_launch: block larger than 1024 threads");
  if (lds_bytes > 160u * 1024u) return fail(LF_EINVAL, "lf_launch: more than 160 KB of LDS requested");
  hipError_t e = hipModuleLaunchKernel(static_cast<hipFunction_t>(fn), gx, gy, gz, bx, by, bz,
                                       lds_bytes, static_cast<hipStream_t>(stream), args, nullptr);
  if (e != hipSuccess) return fail_hip(e, "hipModuleLaunchKernel");
  return 0;
}

int lf_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

int lf_device_info(int dev, char* arch, size_t cap, int* cus, int* lds_bytes) {
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return fail_hip(e, "hipGetDeviceProperties");
  if (arch && cap) {
    std::string a = prop.gcnArchName;
    size_t c = a.find(':');
    if (c != std::string::npos) a = a.substr(0, c);
    size_t n = a.size() < cap - 1 ? a.size() : cap - 1;
    std::memcpy(arch, a.data(), n);
    arch[n] = '\0';
  }
  if (cus) *cus = prop.multiProcessorCount;
  if (lds_bytes) *lds_bytes = static_cast<int>(prop.sharedMemPerBlock);
  return 0;
}

}  // extern "C"
