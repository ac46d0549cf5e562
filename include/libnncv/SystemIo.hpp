// Placeholder kept for source compatibility: the reference header of this name declares nothing
// (include/libnncv/SystemIo.hpp) and examples/Res18/main.cpp includes it.
#ifndef NNCV_LIB_NNCV_RT_SYSTEM_IO_HPP_
#define NNCV_LIB_NNCV_RT_SYSTEM_IO_HPP_
#include "libnncv/DataType.hpp"
#endif
