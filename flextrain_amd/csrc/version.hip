// Library identification string.
#include "common.h"
#include "flexhip.h"

extern "C" const char* fx_version(void) { return "flexhip 0.1 gfx950"; }
