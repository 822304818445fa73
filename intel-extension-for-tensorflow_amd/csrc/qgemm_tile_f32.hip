// Instantiates the MFMA tile kernels for one output type.
#include "qgemm_tile.hpp"

namespace itexhip {
template int dispatch_tile<ITEXHIP_FLOAT>(const uint8_t*, uint32_t, const uint8_t*, int, int, int, const EpilogueArgs&, void*,
                               hipStream_t);
template int dispatch_tile_conv<ITEXHIP_FLOAT>(const uint8_t*, uint32_t, const uint8_t*, int, int, int, const EpilogueArgs&, void*,
                                    hipStream_t, const ConvTileArgs&);
}  // namespace itexhip
