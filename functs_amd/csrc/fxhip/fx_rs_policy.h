// What a generated row-stream translation unit (spec/fx_rs_<key>.hip) includes: the device
// skeleton with its run-time accessors, then the scalar instruction set.  The CPU test harness
// (tests/support/fx_rs_host.cpp) defines FX_RS_HOST and its own accessors before it includes a
// generated unit, which then compiles as plain C++.
#pragma once
#ifndef FX_RS_HOST
#include "fx_rowstream.h"
#endif
#include "fx_rs_ops.h"
