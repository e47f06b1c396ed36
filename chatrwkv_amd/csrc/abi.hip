#include "common.h"

extern "C" int rwkv_abi_version(void) { return 3; }
