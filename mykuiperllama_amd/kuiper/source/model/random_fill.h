// Seeded random tensors written straight into GPU memory, for models that are benchmarked with
// random-init weights of a named architecture (there is no checkpoint to read then).  Element i of
// a tensor is a function of (seed, i) alone — SplitMix64 of seed + i — so a fill does not depend on
// the launch geometry.
#ifndef KUIPER_SOURCE_MODEL_RANDOM_FILL_H
#define KUIPER_SOURCE_MODEL_RANDOM_FILL_H

#include <cstddef>
#include <cstdint>

namespace model {

// n uniform 32-bit words (eight uniform int4 codes each)
void fill_random_words(int32_t* device_ptr, size_t n, uint64_t seed, void* stream);
// n fp16 values uniform on [low, high)
void fill_uniform_fp16(uint16_t* device_ptr, size_t n, uint64_t seed, float low, float high, void* stream);
// n bf16 values mean + std * N(0, 1)  (Box-Muller on two draws per element)
void fill_normal_bf16(uint16_t* device_ptr, size_t n, uint64_t seed, float mean, float std, void* stream);

}  // namespace model

#endif  // KUIPER_SOURCE_MODEL_RANDOM_FILL_H
