# find_package(turbofno): the imported target turbofno::turbofno (libturbofno.so + include/turbofno.h)
include(${CMAKE_CURRENT_LIST_DIR}/turbofnoTargets.cmake)
