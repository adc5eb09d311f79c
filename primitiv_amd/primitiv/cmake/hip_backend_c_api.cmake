# C-API constructors of the HIP backend (primitivCreateHipDevice, ...).
#
# Included from primitiv/CMakeLists.txt inside if(PRIMITIV_BUILD_C_API), after
# the blocks that add the other backends' constructors (lines 285-325) and
# before `add_library(primitiv_c ...)` (line 327):
#     if(PRIMITIV_USE_HIP)
#       include(${PRIMITIV_HIP_BACKEND_DIR}/primitiv/cmake/hip_backend_c_api.cmake)
#     endif()
# The objects go into primitiv_c_all_OBJS, i.e. into libprimitiv_c, like
# primitiv_c_cuda_OBJS: PRIMITIV_C_HANDLE_EXCEPTIONS needs the C API's error
# handler (primitiv/c/internal/internal.cc), which lives in that library.
# hip_backend.cmake must have been included before (it sets the directories).

file(GLOB primitiv_c_hip_HDRS "${PRIMITIV_HIP_BACKEND_DIR}/primitiv/c/devices/hip/*.h")
file(GLOB primitiv_c_hip_SRCS "${PRIMITIV_HIP_BACKEND_DIR}/primitiv/c/devices/hip/*.cc")
install(
  FILES ${primitiv_c_hip_HDRS}
  DESTINATION include/primitiv/c/devices/hip)

add_library(primitiv_c_hip_OBJS OBJECT
  ${primitiv_c_hip_HDRS}
  ${primitiv_c_hip_SRCS}
)
target_include_directories(primitiv_c_hip_OBJS PRIVATE
  ${PRIMITIV_HIP_BACKEND_DIR} ${PRIMITIV_HIP_PHIP_INCLUDE_DIR})
list(APPEND primitiv_c_all_OBJS $<TARGET_OBJECTS:primitiv_c_hip_OBJS>)
