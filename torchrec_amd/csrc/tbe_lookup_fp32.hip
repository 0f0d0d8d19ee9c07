// Instantiates the lookup kernels for TRA_FP32 rows (see tbe_lookup_impl.h).
#include "tbe_lookup_impl.h"

namespace tra {
TRA_DEFINE_LAUNCH(TRA_FP32)
}  // namespace tra
