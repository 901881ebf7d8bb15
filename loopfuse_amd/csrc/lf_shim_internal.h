// lf_shim_internal.h — shared between the translation units of liblf_shim.so (not part of the ABI).
#ifndef LF_SHIM_INTERNAL_H
#define LF_SHIM_INTERNAL_H

#include <string>

// Records `msg` as the calling thread's lf_last_error() text and returns `code`.
int lf_internal_fail(int code, const std::string& msg);

#endif
