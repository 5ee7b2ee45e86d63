// What forward.hip and the translation units of the one-launch forward kernel (forward_single_m.hip)
// both need: the headers of the gate GEMM, the row statistics and the quantiser, and three definitions.
#pragma once
#include "gate_core.hpp"
#include "rows.hpp"
#include "int8_core.hpp"
#include "offsets.hpp"

namespace pm {

constexpr int STATIC_SCRATCH_DEVICES_MAX = 64;

// The first bytes of a forward workspace belong to the one-launch kernel alone (its launch counter,
// ticket counters and published words, forward_single.hpp): its tags are unique only while that
// counter grows by one per launch, so no other entry point may write there.  The tables of the
// two-launch chain and of the stand-alone routing start behind it, whatever the shape.
constexpr size_t FWD_TABLES_OFFSET = 139520;

__device__ __forceinline__ uint64_t lanes_below() { return ((uint64_t)1 << lane_id()) - 1; }

} // namespace pm
