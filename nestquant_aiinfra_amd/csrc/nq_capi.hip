// Library-wide pieces of the C ABI: version and the thread-local error message.
#include "nq_host.h"

namespace nq {

char *error_buffer() {
    static thread_local char buffer[NQ_ERROR_CHARS] = {0};
    return buffer;
}

}  // namespace nq

extern "C" int nq_abi_version(void) { return 2; }

extern "C" const char *nq_last_error(void) { return nq::error_buffer(); }
