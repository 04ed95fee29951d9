// Helpers shared by the C-ABI wrappers: the per-thread error text and the
// try/catch frame that turns C++ exceptions into status codes
// (0 ok, 1 std::exception, 2 anything else). Same convention as
// mops/include/mops/capi.hpp:13-25 and mops/src/capi.cpp:4-12 of
// lab-cosmo/mops.
#ifndef MOPS_CAPI_HELPERS_HPP
#define MOPS_CAPI_HELPERS_HPP

#include <string>

#include "mops/exports.h"

namespace mops {
/// Remember `message` as the calling thread's last error.
void store_error_message(std::string message);
/// The calling thread's last error; valid until the next error on this thread.
MOPS_EXPORT const std::string& get_last_error_message();
} // namespace mops

#define MOPS_CATCH_EXCEPTIONS_BEGIN try {

#define MOPS_CATCH_EXCEPTIONS_END                                                                  \
    return 0;                                                                                      \
    }                                                                                              \
    catch (const std::exception& caught) {                                                         \
        mops::store_error_message(caught.what());                                                  \
        return 1;                                                                                  \
    }                                                                                              \
    catch (...) {                                                                                  \
        mops::store_error_message("unknown error");                                                \
        return 2;                                                                                  \
    }

#endif
