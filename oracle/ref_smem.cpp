// Thin C wrapper around the reference's own host-side header src/index/smem_cal.cuh
// (included from the reference tree in place, not copied).  It is the only reference source
// that a host compiler accepts as is; everything else needs nvcc / FAISS-GPU / RAFT.
// TEST INFRASTRUCTURE ONLY.
#include <cstddef>
#include <cstdint>
#include "smem_cal.cuh"

extern "C" {
uint32_t ref_next_power_of_2(uint32_t n) { return cagra::detail::next_power_of_2(n); }
size_t ref_calculate_and_check_smem(uint32_t itopk, uint32_t dim, uint32_t sw, uint32_t deg, uint32_t bitlen) {
    return cagra::detail::calculate_and_check_smem(itopk, dim, sw, deg, bitlen);
}
}
