// The process-wide random generator functions draw from when they are given seed -1
// (mirrors include/nbla/random_manager.hpp:26-55; initial seed 313 as src/nbla/random_manager.cpp).
#ifndef NBLA_RANDOM_MANAGER_HPP_
#define NBLA_RANDOM_MANAGER_HPP_

#include <nbla/singleton_manager.hpp>

#include <random>

namespace nbla {

class NBLA_API RandomManager {
  std::mt19937 rgen_;
  unsigned seed_;
  int count_;

public:
  ~RandomManager();
  std::mt19937 &get_rand_generator();
  unsigned int get_seed() const;
  // Re-creates the generator; count tells extensions that the seed changed.
  void set_seed(unsigned int seed);
  int get_count() const;

private:
  friend SingletonManager;
  RandomManager();
  RandomManager(const RandomManager &) = delete;
  RandomManager &operator=(const RandomManager &) = delete;
};

} // namespace nbla
#endif
