// Element-wise / broadcast / map entry points for int64_t tensors.
#include "elementwise_impl.h"

AM_EW_DEFINE_ENTRY_POINTS(int64_t, i64)
