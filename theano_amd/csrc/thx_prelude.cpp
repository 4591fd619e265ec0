// The device headers under kernels/ as one string, prepended to every
// generated translation unit handed to hipRTC. thx_prelude.inc is produced by
// build.py from those headers.
#include "thx_internal.h"

namespace thx {

const std::string& device_prelude() {
  static const std::string s =
#include "thx_prelude.inc"
      ;
  return s;
}

}  // namespace thx
