// Seeded pseudo-random ints for test data (ark/include/ark/random.hpp, ark/api/random.cpp).
#ifndef ARK_RANDOM_HPP
#define ARK_RANDOM_HPP

namespace ark {

void srand(int seed = -1);  // -1: seed from the clock
int rand();

}  // namespace ark

#endif  // ARK_RANDOM_HPP
