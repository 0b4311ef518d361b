// SMaLL layer API on MI355X: umbrella header (counterpart of the reference's include/small.h).
// Link with -lsmall_hip (smallframework_amd/lib/libsmall_hip.so).  Plain C++17; no HIP headers
// are needed to compile code that uses this API.
#pragma once

#define SMALL_MAJOR_VERSION 1
#define SMALL_MINOR_VERSION 0
#define SMALL_SUB_VERSON 0

#include <stdint.h>

#include "small_hip.h"
#include "small/Buffer.hpp"
#include "small/utils.hpp"
#include "small/buffers.hpp"
#include "small/interface.hpp"
#include "small/interface_1D.hpp"
#include "small/utils/Timer.hpp"
