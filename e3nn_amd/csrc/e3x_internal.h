// Internal declarations shared by the library's translation units.
#pragma once
#include <string>
#include <vector>

#include "../../include/e3x.h"

namespace e3x {

// records the message for e3x_last_error() and returns `code`
int fail(int code, const std::string& msg);

// dense [2l1+1][2l2+1][2l3+1] tensor, cached for the life of the process
const std::vector<double>& wigner_3j(int l1, int l2, int l3);

// stream-ordered zero fill by a plain store kernel (safe to record into a HIP graph)
int fill_zero_bytes(void* p, size_t n_bytes, void* stream);

}  // namespace e3x
