// Library-level entry points of the C ABI.
#include "common.h"

// changes whenever a signature of the C ABI does: a binding made for another number must not call this library
extern "C" int moba_version(void) { return 115; }

extern "C" const char* moba_strerror(int code) {
  switch (code) {
    case moba::MOBA_OK: return "ok";
    case moba::MOBA_ERR_ARG: return "bad argument (null pointer, non-positive size or misaligned buffer)";
    case moba::MOBA_ERR_UNSUPPORTED: return "unsupported configuration (head_dim must be 128, dtype bf16 or fp16)";
    case moba::MOBA_ERR_LAUNCH: return "kernel launch failed";
    case moba::MOBA_ERR_LIMIT: return "size beyond a supported limit (int32 index range, top-k > 64 or chunks per sequence)";
    default: return "unknown error";
  }
}
