// Strided index spaces for the data-movement kernels: the parameter blocks of the reference's
// strided launches (crates/pyvk/csrc/launch.cpp:18-27 and :84-90: up to 4 dims out / a / b, or
// 8 dims out / a) decoded into one plan that the kernels take by value.
#pragma once

#include "common.h"
#include "../../../include/vkt.h"

#include <string>

namespace vkt {

constexpr uint32_t kMaxDims = 8;

// out[sum_d c_d * so[d]] = a[sum_d c_d * sa[d]] over 0 <= c_d < size[d], dims innermost first;
// strides in units of `unit` bytes (the element, or a multiple of it where the layout allows).
struct MovePlan {
  uint64_t out, a;
  uint64_t n;  // product of the sizes (below 2^32)
  uint32_t ndim, unit;
  uint32_t size[kMaxDims];
  int32_t so[kMaxDims], sa[kMaxDims];
  uint32_t fill[4];  // the fill value repeated over 16 bytes
};

// Offsets (in units) of linear index i.
__device__ __forceinline__ void plan_offsets(const MovePlan& p, uint32_t i, int64_t* o, int64_t* a) {
  int64_t oo = 0, aa = 0;
  uint32_t rem = i;
#pragma unroll
  for (uint32_t d = 0; d < kMaxDims; ++d) {
    if (d < p.ndim) {
      const uint32_t s = p.size[d], q = d + 1 < p.ndim ? rem / s : 0u, c = rem - q * s;
      rem = q;
      oo += int64_t(c) * p.so[d];
      aa += int64_t(c) * p.sa[d];
    }
  }
  *o = oo, *a = aa;
}

// Decodes and checks a block; `item` is the element size in bytes (of out; a's may differ for casts:
// strides stay in elements of each side).  Drops dims of size 1 and merges dims that are contiguous
// in both operands.  False with a message if the block is inconsistent.
inline bool plan_from(const uint64_t out, const uint64_t a, uint32_t n, uint32_t ndim, uint32_t max_dims, const uint32_t* size,
                      const int32_t* so, const int32_t* sa, uint32_t item, const char* who, MovePlan* plan,
                      std::string* err) {
  if (ndim > max_dims) {
    *err = std::string(who) + ": more dims than the block holds";
    return false;
  }
  uint64_t count = 1;
  for (uint32_t d = 0; d < ndim; ++d) count *= size[d];
  if (count != n || (ndim == 0 && n != 1)) {
    *err = std::string(who) + ": n is not the product of the sizes";
    return false;
  }
  MovePlan p{};
  p.out = out, p.a = a, p.n = n, p.unit = item;
  for (uint32_t d = 0; d < ndim; ++d) {
    if (size[d] == 1) continue;
    const int32_t sad = sa ? sa[d] : 0;
    if (p.ndim > 0) {
      const uint32_t l = p.ndim - 1;
      if (int64_t(so[d]) == int64_t(p.so[l]) * p.size[l] && int64_t(sad) == int64_t(p.sa[l]) * p.size[l] &&
          uint64_t(p.size[l]) * size[d] < (1ull << 32)) {
        p.size[l] *= size[d];
        continue;
      }
    }
    p.size[p.ndim] = size[d], p.so[p.ndim] = so[d], p.sa[p.ndim] = sad;
    ++p.ndim;
  }
  *plan = p;
  return true;
}

}  // namespace vkt
