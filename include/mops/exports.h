/* Symbol visibility for the mops C ABI and C++ API.
 *
 * The reference generates this header at configure time
 * (mops/CMakeLists.txt:134-149 of lab-cosmo/mops); this build compiles with
 * -fvisibility=hidden and marks the public entry points explicitly, so the
 * macro is written out by hand here. */
#ifndef MOPS_EXPORTS_H
#define MOPS_EXPORTS_H

#if defined(__GNUC__) || defined(__clang__)
#define MOPS_EXPORT __attribute__((visibility("default")))
#else
#define MOPS_EXPORT
#endif

#endif
