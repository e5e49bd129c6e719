// Process-wide seed source for kernels that draw random numbers
// (hetu/impl/random/CPURandomState.{h,cc} of the reference): once seeded, every
// call hands out the next value of a 64-bit Mersenne Twister, so a run is
// reproducible; unseeded, the wall clock is used.
#pragma once

#include <cstdint>

namespace hetu {
namespace impl {

void SetCPURandomSeed(uint64_t seed);   // 0 is ignored
uint64_t GenNextRandomSeed();

} // namespace impl
} // namespace hetu
