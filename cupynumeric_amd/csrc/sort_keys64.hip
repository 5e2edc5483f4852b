// Instantiates the sort kernels for 64-bit keys (one translation unit per key width so
// that the hipcc runs proceed in parallel; the reference splits its instantiations per
// dtype for the same reason, src/cupynumeric/sort/cub_sort.h:21-115).
#include "sort_driver.h"

namespace cpn {

int sort_keys64(int codec, const SortRequest& r)
{
  switch (codec) {
    case CODEC_UNSIGNED: return sort_typed<uint64_t, CODEC_UNSIGNED>(r);
    case CODEC_SIGNED: return sort_typed<uint64_t, CODEC_SIGNED>(r);
    case CODEC_FLOAT: return sort_typed<uint64_t, CODEC_FLOAT>(r);
    case CODEC_COMPLEX: return sort_typed<uint64_t, CODEC_COMPLEX>(r);  // complex64
    default: return CPN_ERR_DTYPE;
  }
}

}  // namespace cpn
