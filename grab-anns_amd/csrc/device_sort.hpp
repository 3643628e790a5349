#pragma once
#include "common.hpp"

namespace grab {
// sorts `padded` (a power of two) 64-bit keys ascending on `st`, without synchronising
int sort_u64_async(uint64_t* d_keys, uint32_t padded, hipStream_t st);
// the same order written to a second buffer; up to 16384 keys of any count are placed by rank counting in one launch
// (equal keys keep their input order), longer inputs (a power of two) are copied and sorted in place
int rank_sort_u64_async(const uint64_t* d_in, uint64_t* d_out, uint32_t n, hipStream_t st);
}  // namespace grab
