// Error reporting and build identification for the kernel library.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[1024] = "";

int vk_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

int vk_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return vk_fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

extern "C" {

const char* vk_last_error(void) { return g_error; }

// Size in bytes of one element of this build (2: bfloat16, 4: float).
int vk_elem_bytes(void) { return VK_ELEM_BYTES; }

// Bumped whenever an exported signature changes; the Python side refuses a
// library whose number differs from its own.
int vk_abi_version(void) { return 13; }

}  // extern "C"
