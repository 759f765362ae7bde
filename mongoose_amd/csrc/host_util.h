// host_util.h -- host helpers shared inside libmongoose_hip.so.
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>

namespace mg {

// fn(job) for job in [0, njobs) on the library's worker threads (up to 16 with the caller); returns when
// all are done.  One region at a time; fn must not start another.
void parallel_jobs(size_t njobs, const std::function<void(size_t)>& fn);
// fn(begin, end) over [0, n) in pieces of `grain`, through parallel_jobs.
void parallel_for(size_t n, size_t grain, const std::function<void(size_t, size_t)>& fn);

// GGUF block_q4_0 rows -> nibble plane + fp16 scale plane (rows*cols/2 + rows*cols/16 bytes).
void repack_q4_0_host(const uint8_t* raw, int rows, int cols, uint8_t* planar);
// blocks [b0, b1) of a matrix of nb blocks, on the calling thread
void repack_q4_0_blocks(const uint8_t* raw, size_t nb, size_t b0, size_t b1, uint8_t* planar);

}  // namespace mg
