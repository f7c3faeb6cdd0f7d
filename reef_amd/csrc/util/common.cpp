#include "util/common.h"

namespace reef {
int log_level() {
    static int lvl = [] {
        const char* e = std::getenv("REEF_LOG_LEVEL");
        return e ? std::atoi(e) : 1;
    }();
    return lvl;
}
}  // namespace reef
