# Build fragment for primitiv's PRIMITIV_USE_HIP option (AMD MI355X, gfx950).
#
# How it plugs into primitiv's own build (primitiv v0.4.0):
#   * top-level CMakeLists.txt, next to the other backend options (lines 13-16):
#       option(PRIMITIV_USE_HIP "Enable the MI355X (gfx950) HIP backend." OFF)
#   * primitiv/config.h.in, next to PRIMITIV_USE_CUDA:
#       #cmakedefine PRIMITIV_USE_HIP
#   * primitiv/CMakeLists.txt, after the CUDA block (lines 125-187), i.e. before
#     libprimitiv is put together (line 251):
#       if(PRIMITIV_USE_HIP)
#         include(${PRIMITIV_HIP_BACKEND_DIR}/primitiv/cmake/hip_backend.cmake)
#       endif()
#     where PRIMITIV_HIP_BACKEND_DIR points at the directory that holds this
#     backend's `primitiv/` and `csrc/` folders and `include/phip.h`.
#   * primitiv/CMakeLists.txt, inside if(PRIMITIV_BUILD_C_API), after the OpenCL
#     block of the C API (lines 313-325), i.e. before libprimitiv_c is put
#     together (line 327):
#       if(PRIMITIV_USE_HIP)
#         include(${PRIMITIV_HIP_BACKEND_DIR}/primitiv/cmake/hip_backend_c_api.cmake)
#       endif()
#
# This fragment builds libphip (HIP device code, gfx950 only) with hipcc and
# adds the host-side devices::HIP class to the object list that primitiv folds
# into libprimitiv.  The C-API constructors belong to libprimitiv_c, whose
# object list is only created later in primitiv's build: they are added by
# hip_backend_c_api.cmake.

if(NOT DEFINED PRIMITIV_HIP_BACKEND_DIR)
  get_filename_component(PRIMITIV_HIP_BACKEND_DIR "${CMAKE_CURRENT_LIST_DIR}/../.." ABSOLUTE)
endif()
if(NOT DEFINED PRIMITIV_HIP_PHIP_INCLUDE_DIR)
  get_filename_component(PRIMITIV_HIP_PHIP_INCLUDE_DIR "${PRIMITIV_HIP_BACKEND_DIR}/../include" ABSOLUTE)
endif()
if(NOT DEFINED ROCM_PATH)
  set(ROCM_PATH "/opt/rocm")
endif()
find_program(PRIMITIV_HIPCC hipcc HINTS "${ROCM_PATH}/bin" REQUIRED)

set(phip_SRCS
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_runtime.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_elementwise.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_pointwise_unary.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_pointwise_binary.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_indexing.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_reduce.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_random.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_f32.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_f32_direct.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_f32_tile16.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_f32_lds.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_f32_slab.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_f32_rankk.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_f32_pair.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_f32_stream_pair.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_lanes.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_conv_pool.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_h16.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_h16_big.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_gemm_h16_skinny.hip
  ${PRIMITIV_HIP_BACKEND_DIR}/csrc/phip_matmul.hip
)
file(GLOB phip_HDRS "${PRIMITIV_HIP_BACKEND_DIR}/csrc/*.h" "${PRIMITIV_HIP_PHIP_INCLUDE_DIR}/phip.h")
set(phip_FLAGS --offload-arch=gfx950 -O3 -std=c++17 -fPIC
  -Xclang -target-feature -Xclang -packed-fp32-ops)
set(phip_LIB ${CMAKE_CURRENT_BINARY_DIR}/libphip.so)
file(MAKE_DIRECTORY ${CMAKE_CURRENT_BINARY_DIR}/phip)
set(phip_OBJS)
foreach(phip_src ${phip_SRCS})
  get_filename_component(phip_name ${phip_src} NAME_WE)
  set(phip_obj ${CMAKE_CURRENT_BINARY_DIR}/phip/${phip_name}.o)
  add_custom_command(
    OUTPUT ${phip_obj}
    COMMAND ${PRIMITIV_HIPCC} ${phip_FLAGS} -c ${phip_src} -o ${phip_obj}
    DEPENDS ${phip_src} ${phip_HDRS}
    COMMENT "hipcc ${phip_name}.hip (gfx950)"
  )
  list(APPEND phip_OBJS ${phip_obj})
endforeach()
add_custom_command(
  OUTPUT ${phip_LIB}
  COMMAND ${PRIMITIV_HIPCC} --offload-arch=gfx950 -shared -fPIC -o ${phip_LIB} ${phip_OBJS}
  DEPENDS ${phip_OBJS}
  COMMENT "Linking libphip (HIP kernels for gfx950)"
)
add_custom_target(phip ALL DEPENDS ${phip_LIB})
install(FILES ${phip_LIB} DESTINATION lib)
install(FILES ${PRIMITIV_HIP_PHIP_INCLUDE_DIR}/phip.h DESTINATION include)

# Host-side device class (plain C++11, compiled by the project's compiler).
file(GLOB primitiv_hip_HDRS "${PRIMITIV_HIP_BACKEND_DIR}/primitiv/devices/hip/*.h")
file(GLOB primitiv_hip_SRCS "${PRIMITIV_HIP_BACKEND_DIR}/primitiv/devices/hip/*.cc")
add_library(primitiv_hip_OBJS OBJECT ${primitiv_hip_HDRS} ${primitiv_hip_SRCS})
target_include_directories(primitiv_hip_OBJS PRIVATE
  ${PRIMITIV_HIP_BACKEND_DIR} ${PRIMITIV_HIP_PHIP_INCLUDE_DIR})
add_dependencies(primitiv_hip_OBJS phip)
list(APPEND primitiv_all_OBJS $<TARGET_OBJECTS:primitiv_hip_OBJS>)
list(APPEND primitiv_all_DEPS ${phip_LIB})
install(FILES ${primitiv_hip_HDRS} DESTINATION include/primitiv/devices/hip)
