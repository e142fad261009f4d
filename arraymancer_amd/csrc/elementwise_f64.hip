// Element-wise / broadcast / map entry points for double tensors.
#include "elementwise_impl.h"

AM_EW_DEFINE_ENTRY_POINTS(double, f64)
AM_EW_DEFINE_FLOAT_ENTRY_POINTS(double, f64)
