// Error reporting and version of the swin3d_amd C-ABI library.
#include "s3d_common.h"

namespace s3d {

char *error_buffer()
{
    static thread_local char buffer[kErrorBufferBytes] = {0};
    return buffer;
}

}  // namespace s3d

extern "C" __attribute__((visibility("default"))) int s3d_version(void) { return 200; }

extern "C" __attribute__((visibility("default"))) const char *s3d_last_error_string(void) { return s3d::error_buffer(); }
