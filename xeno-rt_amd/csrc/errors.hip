// Last-error text of the calling thread, and the constants that callers must share with the kernels.
#include "cache_layout.h"
#include "xrt_hip.h"

static thread_local char last_error_text[1024] = "";

void xrt_set_error(const char* format, ...) {
    va_list arguments;
    va_start(arguments, format);
    vsnprintf(last_error_text, sizeof(last_error_text), format, arguments);
    va_end(arguments);
}

extern "C" const char* xrt_last_error(void) { return last_error_text; }

extern "C" int xrt_block_tokens(void) { return XRT_BLOCK_TOKENS; }

extern "C" int xrt_cache_key_offset(int token, int dim, int head_dim) { return cache_key_offset(token, dim, head_dim); }
extern "C" int xrt_cache_value_offset(int dim, int token, int head_dim) { return cache_value_offset(dim, token, head_dim); }
