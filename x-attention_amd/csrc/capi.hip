// Library-level entry points of libxattn_hip.so.
#include "xattn_hip.h"

extern "C" int xattn_abi_version(void) { return 1; }

extern "C" const char* xattn_error_string(int code) {
  switch (code) {
    case XATTN_OK: return "ok";
    case XATTN_ERR_NULL: return "a required pointer is null";
    case XATTN_ERR_HEAD_DIM: return "head_dim must be 128";
    case XATTN_ERR_HEADS: return "num_heads must be a positive multiple of num_kv_heads";
    case XATTN_ERR_SHAPE: return "length, block count or pitch out of range";
    case XATTN_ERR_ALIGN: return "pointers must be 16-byte aligned and strides multiples of 8 elements";
    case XATTN_ERR_STRIDE: return "antidiagonal stride must be 4, 8 or 16 and block_size 128";
    case XATTN_ERR_WORKSPACE: return "workspace too small";
    case XATTN_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown error code";
  }
}
