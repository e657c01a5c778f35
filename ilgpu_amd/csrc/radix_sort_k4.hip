// Radix sort of 4-byte keys: instantiates radix_sort_impl.hpp for every value size.
#include "radix_sort_impl.hpp"

namespace ilgpu_hip {

int32_t launch_sort_key_bytes_4(hipStream_t stream, const SortArgs& a) {
  return launch_value<4>(stream, a);
}

}  // namespace ilgpu_hip

