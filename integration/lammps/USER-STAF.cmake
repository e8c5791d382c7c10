# Build glue for LAMMPS' USER-STAF package (lammps/USER-STAF/pair_staf.{h,cpp}, fix_staf.{h,cpp} of the reference)
# against libstaf_hip.so.  Not exercised in this repository (no LAMMPS sources in the build image).
#
# The package sources need no change: pair_staf.cpp includes "staf.h" and calls staf_options_default, staf_load,
# staf_compute and staf_free (lammps/USER-STAF/pair_staf.cpp:152-256); include/staf.h of this repository declares
# those with the reference's argument lists and return codes.
#
# Use: place the block below in cmake/Modules/Packages/USER-STAF.cmake in place of the find of the reference's
# libstaf (that file is included after the `lammps` target exists, which the target_* commands below need; this file
# cannot serve as an initial-cache script for `cmake -C`), then configure with
#
#   cmake -D STAF_HIP_DIR=<checkout of this repository> -D PKG_USER-STAF=on ../cmake
#
if(NOT DEFINED STAF_HIP_DIR)
  message(FATAL_ERROR "set STAF_HIP_DIR to a checkout in which `python -m alphanesgpu_amd.build` has been run")
endif()
find_library(STAF_HIP_LIB NAMES staf_hip PATHS ${STAF_HIP_DIR}/alphanesgpu_amd/lib NO_DEFAULT_PATH REQUIRED)
target_include_directories(lammps PRIVATE ${STAF_HIP_DIR}/include)
target_link_libraries(lammps PRIVATE ${STAF_HIP_LIB})
# the library finds the ROCm runtime through its own DT_NEEDED entries; keep its directory on the run path
set_property(TARGET lammps APPEND PROPERTY BUILD_RPATH ${STAF_HIP_DIR}/alphanesgpu_amd/lib)
set_property(TARGET lammps APPEND PROPERTY INSTALL_RPATH ${STAF_HIP_DIR}/alphanesgpu_amd/lib)
