// Stream-style logging macros of the SWC API (reference: src/SWLOG.h:21-58).
// SWLOG_DEBUG(n) prints when n <= the compile-time LEVELDEBUG (default 0: off).
#ifndef SWC_SWLOG_H_
#define SWC_SWLOG_H_
#include <iostream>

#ifndef LEVELDEBUG
#define LEVELDEBUG 0
#endif

namespace swc {
struct NullStream {
    template <typename T> NullStream &operator<<(const T &) { return *this; }
    NullStream &operator<<(std::ostream &(*)(std::ostream &)) { return *this; }
};
} // namespace swc

#define SWLOG_INFO std::cout << "[INFO] "
#define SWLOG_ERROR std::cerr << "[ERROR] " << __FILE__ << ":" << __LINE__ << " "
#define SWLOG_DEBUG(level)                                                     \
    if ((level) > LEVELDEBUG) {                                                \
    } else                                                                     \
        std::cout << "[DEBUG " << (level) << "] "
#endif
