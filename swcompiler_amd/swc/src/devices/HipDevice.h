// Description of the one device the HIP target generates code for.  The
// reference's src/devices/ holds only an empty DeviceTopology skeleton
// (src/devices/DeviceTopology.h:16-24).  This header is the single place the
// MI355X's figures are written down: the code generator and the placement pass
// read it at compile time (arena alignment, memory size), and libswc_hip
// includes the same header for what its kernels and planners assume (XCD count
// of the workgroup renumbering, LDS budget of the tile shapes, the CU count its
// split plans fall back to, the architecture it accepts at swc_hip_init).
#ifndef SWC_HIP_DEVICE_H_
#define SWC_HIP_DEVICE_H_
#include <cstddef>

namespace swc {
namespace devices {

struct HipDevice {
    static constexpr const char *arch = "gfx950";
    static constexpr int xcds = 8;                        // dies, each with its own L2; workgroups are dealt to them round-robin
    static constexpr int computeUnits = 256;              // 8 XCDs x 32 CUs (a partitioned device reports fewer at run time)
    static constexpr int wavefront = 64;
    static constexpr size_t ldsBytesPerCU = 160 * 1024;   // upper bound of a workgroup's tile ring
    static constexpr size_t hbmBytes = 288ull << 30;      // HBM3E: a program whose arena exceeds this is refused
    // Every tensor starts on a 256-byte boundary of the arena (and swc_hip_malloc
    // returns such addresses): 128-bit vector loads need 16, a full HBM channel
    // interleave granule is 256.
    static constexpr size_t arenaAlignment = 256;
};

} // namespace devices
} // namespace swc
#endif
