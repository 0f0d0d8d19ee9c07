// Instantiates the lookup kernels for TRA_INT8 rows (see tbe_lookup_impl.h).
#include "tbe_lookup_impl.h"

namespace tra {
TRA_DEFINE_LAUNCH(TRA_INT8)
TRA_DEFINE_LAUNCH(TRA_INT8 + kSplitHeader)
}  // namespace tra
