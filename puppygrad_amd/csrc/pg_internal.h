// Declarations shared by the host-side translation units of libpuppygrad_hip.so
// (not part of the public contract in include/puppygrad_hip.h).
#pragma once

#include <string>

#include "../../include/puppygrad_hip.h"

namespace pgh {

// Vectors a kernel stages in LDS (a LayerNorm row, the input of a matrix-vector product, the
// scores of the generic attention kernel) take this many floats at most: 64 KiB of dynamic LDS
// less the kernels' small static blocks.
constexpr unsigned long long kMaxStagedFloats = 16320;

// Records `msg` as the calling thread's last error message and returns `s`.
__attribute__((visibility("hidden"))) pg_status fail(pg_status s, const std::string& msg);

// Gpt2Config::validate (src/models/gpt2/rust.rs:60-95) plus this backend's limits.
__attribute__((visibility("hidden"))) pg_status validate_config(const pg_gpt2_config& c);

}  // namespace pgh
