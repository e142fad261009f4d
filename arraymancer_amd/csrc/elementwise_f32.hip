// Element-wise / broadcast / map entry points for float tensors.
#include "elementwise_impl.h"

AM_EW_DEFINE_ENTRY_POINTS(float, f32)
AM_EW_DEFINE_FLOAT_ENTRY_POINTS(float, f32)
