// Prints the block layout of the ring all-reduce (tirocinio-triennale_amd/host/allreduce_ring.hpp)
// for "<equal|seg> <count> <ranks>": one line "offset count" per block, then "padded max_count".
// Host logic only; no GPU call is made.
#include <cstdio>
#include <cstdlib>
#include <string>

#include "../../tirocinio-triennale_amd/host/allreduce_ring.hpp"

int main(int argc, char **argv)
{
    if (argc != 4) return 2;
    const std::string kind = argv[1];
    const size_t count = std::strtoull(argv[2], nullptr, 10);
    const int ranks = std::atoi(argv[3]);
    const homcomp::RingBlocks b = kind == "seg" ? homcomp::ring_blocks_seg(count, ranks) : homcomp::ring_blocks_equal(count, ranks);
    for (int i = 0; i < ranks; ++i) std::printf("%zu %zu\n", b.offset[(size_t)i], b.count[(size_t)i]);
    std::printf("%zu %zu\n", b.padded, b.max_count);
    return 0;
}
