// Limits of the kernels that their launchers check on the host (plain C++: the host test shim includes this too).
#pragma once

#include <stdint.h>

namespace vkt {

// mma_stream's per-lane offsets into an operand tile are 32-bit: row r <= 255 of a tile lies r * ld bytes past the
// tile's first row, plus a chunk offset and the bias that keeps the offsets non-negative.  Row strides beyond that
// (a wide row-stride view) stay on the tile kernel, which computes these addresses in 64 bits.
constexpr bool mma_stream_strides_ok(uint64_t lda, uint64_t ldb) {
  return 255 * (lda > ldb ? lda : ldb) + 4096 < (1ull << 32);
}

}  // namespace vkt
