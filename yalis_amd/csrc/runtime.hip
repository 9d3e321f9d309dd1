// What every library of kernels carries: the error slot behind yk_last_error() and the
// version that the bindings check (each library is built and loaded on its own, so each has
// its own copy of this file).
#include "common.h"

std::string& yk_error_slot() {
  static thread_local std::string s;
  return s;
}
int yk_fail(const std::string& msg) {
  yk_error_slot() = msg;
  return -1;
}
int yk_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return yk_fail(std::string(what) + ": " + hipGetErrorString(e));
  return 0;
}
extern "C" const char* yk_last_error() { return yk_error_slot().c_str(); }
extern "C" int yk_abi_version() { return 16; }
