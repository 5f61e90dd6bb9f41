// Status strings and ABI version of libpikv_hip.so.
#include "common.hpp"

extern "C" const char* pikv_status_string(int status) {
  switch (status) {
    case PIKV_OK: return "ok";
    case PIKV_ERR_NULL: return "a required pointer is NULL";
    case PIKV_ERR_SHAPE: return "a dimension is out of range";
    case PIKV_ERR_UNSUPPORTED: return "request not supported by this build";
    case PIKV_ERR_WORKSPACE: return "workspace too small";
    case PIKV_ERR_LAUNCH: return "HIP launch failed";
  }
  return "unknown status";
}

extern "C" int pikv_abi_version(void) { return 1003; }  // 1.3: + pikv_quant8_minshift, pikv_decode_attend, pikv_stream_probe
