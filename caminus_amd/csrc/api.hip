// Library-level entry points of the C ABI: version, error strings.
#include "common.cuh"

extern "C" {
int camx_version(void) { return 1; }
const char * camx_error_string(int err) { return hipGetErrorString((hipError_t)err); }
const char * camx_arch(void) { return "gfx950"; }
}
