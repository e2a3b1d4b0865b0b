// PackTraits<DataT> (register packing ratios) is defined with the types; this header keeps the
// reference's include path (pack_util.hpp:42-53) working.
#ifndef ROCWMMA_PACK_UTIL_HPP
#define ROCWMMA_PACK_UTIL_HPP

#include "types.hpp"

#endif // ROCWMMA_PACK_UTIL_HPP
