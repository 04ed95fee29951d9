/* Umbrella header of the mops C ABI: 60 operation entry points plus the
 * error-text accessor (replaces mops/include/mops.h:1-22 of lab-cosmo/mops),
 * and the AMD-specific additions of mops/amd.h. */
#ifndef MOPS_H
#define MOPS_H

#include "mops/exports.h"
#include "mops/hpe.h"
#include "mops/opsa.h"
#include "mops/opsaw.h"
#include "mops/sap.h"
#include "mops/sasaw.h"
#include "mops/amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Text of the last error raised on the calling thread by any mops_* function.
 * The pointer stays valid until the next failing call on the same thread. */
MOPS_EXPORT const char* mops_get_last_error_message(void);

#ifdef __cplusplus
}
#endif

#endif
