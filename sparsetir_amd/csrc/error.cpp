// Last-error storage behind stir_last_error().
#include "common.h"
#include "../../include/sparsetir_amd.h"

#include <string>

namespace stir {
namespace {
thread_local std::string g_last_error;
}

void set_error(const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
}

const char* get_error() { return g_last_error.c_str(); }
}  // namespace stir

extern "C" {
const char* stir_last_error(void) { return stir::get_error(); }
const char* stir_version(void) { return "sparsetir_amd 0.1 (gfx950)"; }
}
