// Error text and version of the C ABI.
#include "common.cuh"

namespace xad {
char* last_error_buffer() {
    static thread_local char buffer[kLastErrorCapacity] = {0};
    return buffer;
}
}  // namespace xad

extern "C" const char* xad_last_error(void) { return xad::last_error_buffer(); }
extern "C" int xad_abi_version(void) { return 1; }

#ifndef XAD_SOURCE_DIGEST
#define XAD_SOURCE_DIGEST ""
#endif
extern "C" const char* xad_source_digest(void) { return XAD_SOURCE_DIGEST; }
