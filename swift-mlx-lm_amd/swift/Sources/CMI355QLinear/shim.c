/* SwiftPM wants at least one source file in a C target. */
#include "include/shim.h"
