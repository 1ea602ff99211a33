// Library version, the offload architecture and the hash of the sources the library was built from
// (MOR_SRC_HASH comes from the build script; a binding compares it with the sources it sits next to).
#include "../../include/mor_hip.h"

#ifndef MOR_SRC_HASH
#define MOR_SRC_HASH "unknown"
#endif

extern "C" const char* mor_version(void) { return "mor_hip 0.2 (gfx950) src " MOR_SRC_HASH; }
