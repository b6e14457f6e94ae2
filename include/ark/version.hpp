// Version of the ark:: API served (ark/include/ark/version.hpp).
#ifndef ARK_VERSION_HPP
#define ARK_VERSION_HPP

#include <string>

#define ARK_MAJOR 0
#define ARK_MINOR 5
#define ARK_PATCH 0
#define ARK_VERSION (ARK_MAJOR * 10000 + ARK_MINOR * 100 + ARK_PATCH)

namespace ark {

// Version string of the backend library.
std::string version();

}  // namespace ark

#endif  // ARK_VERSION_HPP
