// Host-side copy into pinned staging memory on a few threads (the reference ABI hands over pageable host buffers:
// examples/Res18/main.cpp:79-99).  One thread moves about 10 GB/s, which for config 4's 9.6 MB input is three times
// the forward pass; four threads bring the staging copy under the time the DMA engine needs for the same bytes.
#pragma once
#include <cstddef>

namespace nncv_hip {

// dst[0..bytes) = src[0..bytes), split over the calling thread and the pool's workers (started on first use, kept for the
// life of the process, asleep between calls).  Callers are serialised by the library's mutex.
void parallel_copy(void* dst, const void* src, size_t bytes);

}  // namespace nncv_hip
