// host_util.h -- host helpers shared inside libmongoose_hip.so.
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>

namespace mg {

// fn(begin, end) over [0, n) on up to 16 host threads, in pieces of `grain`.
void parallel_for(size_t n, size_t grain, const std::function<void(size_t, size_t)>& fn);

// GGUF block_q4_0 rows -> nibble plane + fp16 scale plane (rows*cols/2 + rows*cols/16 bytes).
void repack_q4_0_host(const uint8_t* raw, int rows, int cols, uint8_t* planar);

}  // namespace mg
