// Umbrella header of the mops C++ API (replaces mops/include/mops.hpp:1-13
// of lab-cosmo/mops).
#ifndef MOPS_HPP
#define MOPS_HPP

#include "mops/exports.h"

#include "mops/capi.hpp"
#include "mops/hpe.hpp"
#include "mops/opsa.hpp"
#include "mops/opsaw.hpp"
#include "mops/sap.hpp"
#include "mops/sasaw.hpp"

#endif
