// Element-wise / broadcast / map entry points for int32_t tensors.
#include "elementwise_impl.h"

AM_EW_DEFINE_ENTRY_POINTS(int32_t, i32)
