// Instantiates the lookup kernels for TRA_FP16 rows (see tbe_lookup_impl.h).
#include "tbe_lookup_impl.h"

namespace tra {
TRA_DEFINE_LAUNCH(TRA_FP16)
}  // namespace tra
