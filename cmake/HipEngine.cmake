# The MI355X HIP engine as a fourth engine of the Visual Mesh library, switched like the reference's OpenCL and Vulkan
# engines (reference cpp/CMakeLists.txt:30-53): include this file from cpp/CMakeLists.txt after the `visualmesh` target
# exists.
#
#   -DBUILD_HIP_ENGINE=ON                      use the engine; needs the C ABI library and its header:
#   -DVISUALMESH_HIP_ROOT=<this repository>    include/visualmesh_hip.h, visualmesh_amd/lib/libvisualmesh_hip.so
#                                              (built with `python -m visualmesh_amd.build`: hipcc --offload-arch=gfx950)
#   BUILD_HIP_ENGINE=OFF (default)             defines VISUALMESH_DISABLE_HIP: engine/hip/engine.hpp is then empty and
#                                              call sites are written as
#                                                  #if !defined(VISUALMESH_DISABLE_HIP)
#                                                  benchmark<visualmesh::engine::hip::Engine<Scalar>>(...);
#                                                  #endif
option(BUILD_HIP_ENGINE "Build the MI355X HIP engine (gfx950)" OFF)

if(BUILD_HIP_ENGINE)
  set(VISUALMESH_HIP_ROOT "" CACHE PATH "Tree that holds include/visualmesh_hip.h and visualmesh_amd/lib/libvisualmesh_hip.so")
  find_path(VISUALMESH_HIP_INCLUDE_DIR visualmesh_hip.h
            HINTS "${VISUALMESH_HIP_ROOT}/include" "${CMAKE_CURRENT_LIST_DIR}/../include")
  find_library(VISUALMESH_HIP_LIBRARY visualmesh_hip
               HINTS "${VISUALMESH_HIP_ROOT}/visualmesh_amd/lib" "${CMAKE_CURRENT_LIST_DIR}/../visualmesh_amd/lib")
  if(NOT VISUALMESH_HIP_INCLUDE_DIR OR NOT VISUALMESH_HIP_LIBRARY)
    message(FATAL_ERROR "BUILD_HIP_ENGINE is on but visualmesh_hip.h / libvisualmesh_hip.so were not found: "
                        "build them with `python -m visualmesh_amd.build` and set VISUALMESH_HIP_ROOT")
  endif()
  # the engine header itself (host C++14, no device code) when it has not been copied into cpp/visualmesh/engine/hip/
  if(NOT EXISTS "${CMAKE_CURRENT_SOURCE_DIR}/visualmesh/engine/hip/engine.hpp")
    target_include_directories(visualmesh INTERFACE "${CMAKE_CURRENT_LIST_DIR}/../visualmesh_amd/cpp")
  endif()
  target_include_directories(visualmesh INTERFACE "${VISUALMESH_HIP_INCLUDE_DIR}")
  target_link_libraries(visualmesh INTERFACE "${VISUALMESH_HIP_LIBRARY}")
else()
  target_compile_definitions(visualmesh INTERFACE VISUALMESH_DISABLE_HIP)
endif()
