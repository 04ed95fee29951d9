# find_package(mops CONFIG) for the MI355X build of mops.
#
# Defines the imported target `mops`, the name under which the reference
# exports its library (mops/CMakeLists.txt:224-257 and
# mops/cmake/mops-config.in.cmake of lab-cosmo/mops), so that a project which
# does
#
#     find_package(mops CONFIG REQUIRED)
#     target_link_libraries(my_target mops)
#
# gets libmops.so of this package and its headers (mops.h, mops.hpp, mops/*).
# Point CMake here with -Dmops_DIR=<.../mops_amd/cmake/mops> or by adding the
# mops_amd directory to CMAKE_PREFIX_PATH.
#
# Layout this file expects, relative to itself:
#     ../../lib/libmops.so          built by mops_amd/csrc/Makefile
#     ../../include/                 headers inside an installed package, or
#     ../../../include/              headers of the source tree
get_filename_component(_mops_package_dir "${CMAKE_CURRENT_LIST_DIR}/../.." ABSOLUTE)

set(_mops_library "${_mops_package_dir}/lib/libmops.so")
if (NOT EXISTS "${_mops_library}")
    set(mops_FOUND FALSE)
    set(mops_NOT_FOUND_MESSAGE "${_mops_library} does not exist: build it with `make -C mops_amd/csrc`")
    return()
endif()

if (EXISTS "${_mops_package_dir}/include/mops.h")
    set(_mops_include_dir "${_mops_package_dir}/include")
else()
    get_filename_component(_mops_include_dir "${_mops_package_dir}/../include" ABSOLUTE)
endif()
if (NOT EXISTS "${_mops_include_dir}/mops.h")
    set(mops_FOUND FALSE)
    set(mops_NOT_FOUND_MESSAGE "mops.h not found next to ${_mops_package_dir}")
    return()
endif()

if (NOT TARGET mops)
    add_library(mops SHARED IMPORTED)
    set_target_properties(mops PROPERTIES
        IMPORTED_LOCATION "${_mops_library}"
        IMPORTED_SONAME "libmops.so"
        INTERFACE_INCLUDE_DIRECTORIES "${_mops_include_dir}"
    )
endif()

unset(_mops_package_dir)
unset(_mops_library)
unset(_mops_include_dir)
