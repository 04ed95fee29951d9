# Version file for find_package(mops <version> CONFIG): compatible with requests
# for the same major.minor, as the reference's own version file
# (write_basic_package_version_file(... SameMinorVersion), mops/CMakeLists.txt:227-231).
set(PACKAGE_VERSION "0.1.0")

if (PACKAGE_FIND_VERSION)
    if ("${PACKAGE_FIND_VERSION_MAJOR}.${PACKAGE_FIND_VERSION_MINOR}" STREQUAL "0.1")
        set(PACKAGE_VERSION_COMPATIBLE TRUE)
        if ("${PACKAGE_FIND_VERSION}" STREQUAL "${PACKAGE_VERSION}")
            set(PACKAGE_VERSION_EXACT TRUE)
        endif()
    else()
        set(PACKAGE_VERSION_COMPATIBLE FALSE)
    endif()
else()
    set(PACKAGE_VERSION_COMPATIBLE TRUE)
endif()
