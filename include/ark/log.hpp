// Logging entry point of the ark:: API (ark/include/ark/log.hpp:9-14).
#ifndef ARK_LOG_HPP
#define ARK_LOG_HPP

#include <string>

namespace ark {

enum LogLevel { DEBUG = 0, INFO = 1, WARN = 2, ERROR = 3 };

// Writes "ARK <pid> <LEVEL> <file>:<line> <msg>" to the log stream when `level` is at or above
// ARK_LOG_LEVEL (default INFO).  Unlike the reference's ERROR level this never throws: errors are
// raised through the exception classes of error.hpp.
void log(LogLevel level, const std::string &file, int line, const std::string &msg);

}  // namespace ark

#endif  // ARK_LOG_HPP
