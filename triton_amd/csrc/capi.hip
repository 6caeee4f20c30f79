// Library-wide pieces of the C ABI: version, per-thread error string, and host-side evaluation of the
// scalar MX conversions (so their bit-exactness can be checked on a machine without a GPU).
#include <string.h>

#include "mx_math.h"

namespace tk {

static thread_local char g_last_error[512] = "";

int32_t fail(int32_t code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace tk

extern "C" int32_t tk_version(void) { return 100; }

extern "C" const char* tk_last_error(void) { return tk::g_last_error; }

extern "C" int32_t tk_host_mx_convert(const float* in, int64_t n, int32_t kind, uint8_t* out) {
  if (!in || !out || n < 0) return tk::fail(TK_ERR_INVALID, "tk_host_mx_convert: bad argument");
  for (int64_t i = 0; i < n; ++i) {
    if (kind == TK_E2M1)
      out[i] = (uint8_t)tk::e2m1_code(in[i]);
    else if (kind == TK_E4M3)
      out[i] = (uint8_t)tk::e4m3_byte(tk::mx_clamp(in[i], 448.0f));
    else if (kind == TK_E5M2)
      out[i] = (uint8_t)tk::e5m2_byte(tk::mx_clamp(in[i], 57344.0f));
    else
      return tk::fail(TK_ERR_INVALID, "tk_host_mx_convert: bad kind %d", kind);
  }
  return TK_OK;
}

extern "C" int32_t tk_host_mx_scale(const float* absmax, int64_t n, int32_t kind, int32_t rounding, uint8_t* out) {
  if (!absmax || !out || n < 0) return tk::fail(TK_ERR_INVALID, "tk_host_mx_scale: bad argument");
  for (int64_t i = 0; i < n; ++i) out[i] = (uint8_t)(tk::mx_scale_bits(absmax[i], kind, rounding) >> 23);
  return TK_OK;
}
