// ark::init / srand / rand / version (ark/api/init.cpp, random.cpp, version.cpp).
#include <ark/ark.hpp>

#include <cstdlib>
#include <ctime>

#include "../../../include/arkmi.h"
#include "ir.hpp"

namespace ark {

void init() { reload_env(); }

void log(LogLevel level, const std::string &file, int line, const std::string &msg) {
    static const char *names[] = {"DEBUG", "INFO", "WARN", "ERROR"};
    if (level < log_level()) return;
    const int l = level < DEBUG ? DEBUG : level > ERROR ? ERROR : level;
    std::clog << format_message(names[l], file.c_str(), line, msg) << '\n';
}

void srand(int seed) { ::srand(seed < 0 ? (unsigned)::time(nullptr) : (unsigned)seed); }

int rand() { return ::rand(); }

std::string version() { return arkmi_version(); }

}  // namespace ark
