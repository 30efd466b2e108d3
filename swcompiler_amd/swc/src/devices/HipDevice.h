// Description of the one device the HIP target generates code for.  The
// reference's src/devices/ holds only an empty DeviceTopology skeleton
// (src/devices/DeviceTopology.h:16-24); these constants are what the memory
// lowering and the code generator need to know about an MI355X.
#ifndef SWC_HIP_DEVICE_H_
#define SWC_HIP_DEVICE_H_
#include <cstddef>

namespace swc {
namespace devices {

struct HipDevice {
    const char *arch = "gfx950";
    int computeUnits = 256;              // 8 XCDs x 32 CUs
    int xcds = 8;
    int wavefront = 64;
    size_t ldsBytesPerCU = 160 * 1024;
    size_t hbmBytes = 288ull << 30;      // HBM3E
    double hbmBytesPerSec = 8.0e12;
    double fp32MatrixFlops = 157.3e12;   // dense MFMA fp32
    // Every tensor starts on a 256-byte boundary of the arena: 128-bit vector
    // loads need 16, a full HBM channel interleave granule is 256.
    size_t arenaAlignment = 256;
};

} // namespace devices
} // namespace swc
#endif
