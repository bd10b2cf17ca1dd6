// Library-level entry points that need no device code.
#include "ofq.h"

extern "C" const char* ofq_status_string(int status) {
  switch (status) {
    case OFQ_OK: return "ok";
    case OFQ_ERR_NULL_POINTER: return "null pointer (or optional tensor present/absent against `symmetric`)";
    case OFQ_ERR_BAD_DTYPE: return "dtype not valid for this argument";
    case OFQ_ERR_BAD_SHAPE: return "inconsistent sizes";
    case OFQ_ERR_BAD_ATTR: return "attribute outside the op's domain";
    case OFQ_ERR_UNSUPPORTED: return "no kernel covers this combination";
    case OFQ_ERR_WORKSPACE: return "workspace missing or too small";
    case OFQ_ERR_MISALIGNED: return "pointer not 16-byte aligned";
    case OFQ_ERR_LAUNCH: return "kernel launch failed";
    case OFQ_ERR_TOO_LARGE: return "input exceeds the fixed scratch capacity of this entry point";
    default: return "unknown status";
  }
}

extern "C" int ofq_abi_version(void) { return 1; }
