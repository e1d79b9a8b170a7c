// Declarations shared by the host-side translation units of libpuppygrad_hip.so
// (not part of the public contract in include/puppygrad_hip.h).
#pragma once

#include <string>

#include "../../include/puppygrad_hip.h"

namespace pgh {

// Records `msg` as the calling thread's last error message and returns `s`.
__attribute__((visibility("hidden"))) pg_status fail(pg_status s, const std::string& msg);

// Gpt2Config::validate (src/models/gpt2/rust.rs:60-95) plus this backend's limits.
__attribute__((visibility("hidden"))) pg_status validate_config(const pg_gpt2_config& c);

}  // namespace pgh
