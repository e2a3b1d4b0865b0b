// IOConfig<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> lives with the fragment class; this
// header keeps the reference's include path (io_config.hpp:65-113) working.
#ifndef ROCWMMA_IO_CONFIG_HPP
#define ROCWMMA_IO_CONFIG_HPP

#include "../rocwmma.hpp"
#include "io_traits.hpp"

#endif // ROCWMMA_IO_CONFIG_HPP
