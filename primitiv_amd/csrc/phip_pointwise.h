// Shared pieces of the elementwise kernels: 16-byte packs, launch geometry.
#ifndef PHIP_POINTWISE_H_
#define PHIP_POINTWISE_H_

#include "phip_internal.h"
#include "phip_types.h"

namespace phip {
namespace pointwise {

constexpr int kBlock = 256;

// 16 bytes of T: what one lane moves per load/store instruction.
template <typename T>
struct alignas(16) Pack {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

template <typename T>
__device__ inline Pack<T> load_pack(const T *p) {
  return *reinterpret_cast<const Pack<T> *>(p);
}

template <typename T>
__device__ inline void store_pack(T *p, const Pack<T> &v) {
  *reinterpret_cast<Pack<T> *>(p) = v;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Blocks for a grid-stride loop over `items` work items: enough to fill the
// device a few times over, never more than the items need.
inline unsigned blocks_for(size_t items, const phip_ctx *ctx) {
  const size_t blocks = (items + kBlock - 1) / kBlock;
  const size_t cap = (size_t)ctx->prop.multiProcessorCount * 32;
  return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

}  // namespace pointwise
}  // namespace phip

#endif  // PHIP_POINTWISE_H_
