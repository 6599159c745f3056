// ssr_sortscan.hpp -- the sort / scan seam of the backend (src/backend/common/SortScan.h:42-60), for the two
// instantiations the tile-intersection stage uses: sort_pairs<int64_t, int32_t> on a bit range of the key
// (src/kernels/tile/IntersectTile.cu:486-493) and inclusive_sum<int64_t> (:425-431). Same names, argument order
// and meaning as the reference's templates; both forward to the C ABI of libssr_hip.so with working space taken
// from the device pool. Other instantiations are not built and fail at link time, as an uncompiled variant should.
#pragma once
#include <cstdint>

#include "ssr_host_types.hpp"

namespace backend {

// Two device buffers of which `selector` names the one that holds the data; a sort may leave its result in
// either and says which by updating the selector (cub::DoubleBuffer's contract, SortScan.h:42-51).
template <typename T>
struct DoubleBuffer {
    T* buffers[2];
    int selector = 0;

    DoubleBuffer(T* current, T* alternate) : buffers{current, alternate} {}
    T* current() const { return buffers[selector]; }
    T* alternate() const { return buffers[selector ^ 1]; }
};

// Stable LSD radix sort of (key, value) pairs on key bits [begin_bit, end_bit); the keys compare as unsigned.
// The alternate buffers are working space; afterwards keys.current() / values.current() hold the result.
template <typename KeyT, typename ValueT>
void sort_pairs(DoubleBuffer<KeyT>& keys, DoubleBuffer<ValueT>& values, int64_t num_items, int begin_bit, int end_bit,
                Stream stream = kDefaultStream);

// out[i] = in[0] + ... + in[i]; in == out is allowed.
template <typename T>
void inclusive_sum(const T* in, T* out, int64_t num_items, Stream stream = kDefaultStream);

template <>
void sort_pairs<int64_t, int32_t>(DoubleBuffer<int64_t>& keys, DoubleBuffer<int32_t>& values, int64_t num_items,
                                  int begin_bit, int end_bit, Stream stream);
template <>
void inclusive_sum<int64_t>(const int64_t* in, int64_t* out, int64_t num_items, Stream stream);

}  // namespace backend
