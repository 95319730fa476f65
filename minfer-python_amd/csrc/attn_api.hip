// Entry points of the C ABI that are not tied to one operator.
#include "attn_host.h"


MINFER_ATTN_EXPORT int minfer_attn_version(void) { return 1000; }

MINFER_ATTN_EXPORT const char* minfer_attn_last_error(void) { return minfer_attn::error_buf(); }
