// Library-wide initialisation (ark/include/ark/init.hpp, ark/api/init.cpp:15-19).
#ifndef ARK_INIT_HPP
#define ARK_INIT_HPP

namespace ark {

// Reads the ARK_* environment variables again (they are otherwise read once, on first use).
void init();

}  // namespace ark

#endif  // ARK_INIT_HPP
