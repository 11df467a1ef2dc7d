// Error reporting for the C interface: the last refusal's message, per thread.
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[1024] = "";

void holon_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
}

extern "C" const char* holon_last_error(void) { return g_error; }
extern "C" int holon_abi_version(void) { return 1; }
