// Library-level entry points: ABI version and the per-thread error string.
#include "common.h"

extern "C" int acache_abi_version(void) { return ACACHE_ABI_VERSION; }

extern "C" const char *acache_last_error(void) { return acache::err_buf(); }
