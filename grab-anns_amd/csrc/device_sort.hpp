#pragma once
#include "common.hpp"

namespace grab {
// sorts `padded` (a power of two) 64-bit keys ascending on `st`, without synchronising
int sort_u64_async(uint64_t* d_keys, uint32_t padded, hipStream_t st);
}  // namespace grab
