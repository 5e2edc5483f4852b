// Instantiates the sort kernels for 128-bit keys (complex128).  One translation unit per key
// width keeps the hipcc runs parallel; the reference has one per dtype for the same reason
// (src/cupynumeric/sort/thrust_sort.h:129-145 declares the complex instantiations).
#include "sort_driver.h"

namespace cpn {

int sort_keys128(int codec, const SortRequest& r)
{
  switch (codec) {
    case CODEC_COMPLEX: return sort_typed<U128, CODEC_COMPLEX>(r);
    default: return CPN_ERR_DTYPE;
  }
}

}  // namespace cpn
