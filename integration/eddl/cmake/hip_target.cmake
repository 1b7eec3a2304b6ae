# BUILD_TARGET=HIP: EDDL's gpu_* seam served by libeddlhip.so (AMD MI355X, gfx950) instead of src/hardware/gpu.
# Included from src/CMakeLists.txt when USE_HIP is ON (see eddl_hip.patch).  No CUDA toolkit, cuBLAS, cuRAND or
# cuDNN is looked for; the only dependency is the backend itself:
#   -D EDDLHIP_ROOT=/path/to/backend   a checkout or install prefix that holds include/eddlhip.h and libeddlhip.so
set(EDDLHIP_ROOT "" CACHE PATH "Checkout or install prefix of the eddlhip backend (include/eddlhip.h, libeddlhip.so)")

find_path(EDDLHIP_INCLUDE_DIR eddlhip.h HINTS ${EDDLHIP_ROOT} PATH_SUFFIXES include)
find_library(EDDLHIP_LIBRARY eddlhip HINTS ${EDDLHIP_ROOT} PATH_SUFFIXES lib lib64 eddl_amd)
if(NOT EDDLHIP_INCLUDE_DIR OR NOT EDDLHIP_LIBRARY)
    message(FATAL_ERROR "BUILD_TARGET=HIP needs the eddlhip backend: set -D EDDLHIP_ROOT=<path holding include/eddlhip.h and libeddlhip.so>")
endif()

# HIP_HEADERS / HIP_SOURCES are globbed (and taken out of the common file list) in src/CMakeLists.txt:
#   include/eddl/hardware/hip/hip_backend.h
#   src/hardware/hip/hip_backend.cpp   the gpu_* functions of the forward path, eddl::build and eddl::predict
#   src/hardware/hip/hip_stubs.cpp     every other gpu_* declaration (raises through msg())
target_sources(${PROJECT_NAME} PRIVATE ${HIP_HEADERS} ${HIP_SOURCES})
target_include_directories(${PROJECT_NAME} PRIVATE ${EDDLHIP_INCLUDE_DIR})
target_link_libraries(${PROJECT_NAME} PRIVATE ${EDDLHIP_LIBRARY})
message(STATUS "HIP backend: ${EDDLHIP_LIBRARY}")
