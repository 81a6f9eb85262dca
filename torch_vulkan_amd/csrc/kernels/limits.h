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

// K cut into slices over workgroups: `chunks` chunks in slices of ceil(chunks / wanted) each leave the last of `wanted`
// slices empty where that does not divide (65 chunks in 16 slices of 5 fill 13).  The kernels count a slice's chunks
// as (end - begin) in unsigned arithmetic, so a launcher must never make an empty one: this is the count it launches.
struct KSlices {
  uint32_t slices, chunks_per_slice;
};
constexpr KSlices k_slices(uint32_t chunks, uint32_t wanted) {
  const uint32_t want = wanted < 1 ? 1 : (wanted > chunks && chunks ? chunks : wanted);
  const uint32_t per = chunks ? (chunks + want - 1) / want : 1;
  return KSlices{chunks ? (chunks + per - 1) / per : 1, per};
}

}  // namespace vkt
