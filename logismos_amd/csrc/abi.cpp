// Library identity.
#include "launch_common.hpp"

extern "C" int logismos_decode_abi_version(void) { return 5; }
extern "C" const char* logismos_decode_offload_arch(void) { return "gfx950"; }
