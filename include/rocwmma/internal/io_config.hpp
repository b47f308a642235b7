// The traits existing code takes from <rocwmma/internal/io_config.hpp> (fragment sizes, pack
// ratios) are defined together with the fragment class here; this header keeps the reference's
// include path working and keeps the toolchain's own rocWMMA copy from being picked up instead.
#ifndef ROCWMMA_AMD_FORWARD_IO_CONFIG_HPP
#define ROCWMMA_AMD_FORWARD_IO_CONFIG_HPP

#include "../rocwmma.hpp"

#endif
