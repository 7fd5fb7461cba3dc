// Version and error-text entry points of libtrimkv_hip.so.
#include "common.hip.h"

extern "C" int trimkv_version(void) { return 100; }  // 0.1.0

extern "C" const char* trimkv_last_error(void) { return trimkv::err_buf(); }
