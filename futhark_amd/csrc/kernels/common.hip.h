// The device-side building blocks (operators, wave64 cross-lane primitives,
// 128-bit memory access, launch helpers) live in the public header, so that
// per-program operators can be written against them.
#pragma once
#include "futhark_amd_device.hpp"
