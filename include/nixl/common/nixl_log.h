// Stream-style logging macros with the reference's names (src/utils/common/nixl_log.h:33-95),
// backed by std::cerr instead of abseil.  Level comes from NIXL_LOG_LEVEL
// (ERROR|WARN|INFO|DEBUG|TRACE, default WARN).
#ifndef NIXL_AMD_LOG_H
#define NIXL_AMD_LOG_H

#include <cassert>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <sstream>

namespace nixl_amd_log {

inline int
level() {
    static const int lvl = [] {
        const char *e = std::getenv("NIXL_LOG_LEVEL");
        if (!e) return 1;
        if (!strcasecmp(e, "ERROR")) return 0;
        if (!strcasecmp(e, "WARN")) return 1;
        if (!strcasecmp(e, "INFO")) return 2;
        if (!strcasecmp(e, "DEBUG")) return 3;
        if (!strcasecmp(e, "TRACE")) return 4;
        return 1;
    }();
    return lvl;
}

// Collects one message and emits it on destruction if its level is enabled.
class line {
public:
    line(int lvl, const char *tag) : on_(lvl <= level()) {
        if (on_) os_ << "[nixl " << tag << "] ";
    }
    ~line() {
        if (on_) std::cerr << os_.str() << std::endl;
    }
    template<typename T>
    line &
    operator<<(const T &v) {
        if (on_) os_ << v;
        return *this;
    }

private:
    bool on_;
    std::ostringstream os_;
};

} // namespace nixl_amd_log

#define NIXL_ERROR nixl_amd_log::line(0, "E")
#define NIXL_ERROR_FUNC NIXL_ERROR << __FUNCTION__ << ": "
#define NIXL_WARN nixl_amd_log::line(1, "W")
#define NIXL_INFO nixl_amd_log::line(2, "I")
#define NIXL_DEBUG nixl_amd_log::line(3, "D")
#define NIXL_TRACE nixl_amd_log::line(4, "T")
#define NIXL_ASSERT(x) assert(x)

#endif
