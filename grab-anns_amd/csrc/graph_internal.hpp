// Graph-optimisation helpers shared between the global build and the time-partitioned build.
#pragma once
#include "common.hpp"

namespace grab {

// Reverse lists of the columns [col_lo, col_lo + width) of a graph [num_dataset, degree]: for every
// destination its first `cap` sources (0xFFFFFFFF padding) in the order (column, source) or, with
// by_source, (source, column), and the full in-degree in d_counts.  Synchronises the stream.
int reverse_lists(const uint32_t* d_graph, size_t num_dataset, uint32_t degree, uint32_t col_lo, uint32_t width, int by_source,
                  uint32_t cap, uint32_t* d_rev, uint32_t* d_counts, hipStream_t st);

}  // namespace grab
