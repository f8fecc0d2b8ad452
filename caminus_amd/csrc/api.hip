// Library-level entry points of the C ABI: version, error strings, initialisation.
#include "common.cuh"

__attribute__((visibility("hidden"))) int silu_lut_get(hipStream_t st, const uint16_t ** lut);       // quant.hip
__attribute__((visibility("hidden"))) int dsilu_luts_init(hipStream_t st);                            // actq.hip

extern "C" {
int camx_version(void) { return 2; }
const char * camx_error_string(int err) { return hipGetErrorString((hipError_t)err); }
const char * camx_arch(void) { return "gfx950"; }
// Fills the lookup tables of the current device (bf16(silu g) and the sigmoid of the fused backward, with their LDS extracts) and waits for
// `stream` once. After it no entry point synchronizes or takes the fill path again on this device, so every later call is safe inside a
// stream capture. Calling it again, from any thread, is a no-op; without it the first call of an entry point that needs a table does the same.
int camx_init(hipStream_t stream) {
    const uint16_t * lut = nullptr;
    const int rc = silu_lut_get(stream, &lut);
    return rc ? rc : dsilu_luts_init(stream);
}
}
