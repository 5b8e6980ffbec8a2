// Process-wide singletons with ordered destruction
// (mirrors include/nbla/singleton_manager.hpp).
#ifndef NBLA_SINGLETON_MANAGER_HPP_
#define NBLA_SINGLETON_MANAGER_HPP_

#include <nbla/common.hpp>

#include <functional>
#include <mutex>
#include <typeindex>
#include <unordered_map>

namespace nbla {

class NBLA_API SingletonManager {
public:
  // The single instance of T, created on first use.
  template <typename T> static T *get() {
    SingletonManager &self = get_self();
    std::lock_guard<std::recursive_mutex> lock(self.mtx_);
    const std::type_index key(typeid(T));
    auto it = self.objects_.find(key);
    if (it != self.objects_.end())
      return static_cast<T *>(it->second.first);
    T *obj = new T();
    self.objects_[key] = {obj, [](void *p) { delete static_cast<T *>(p); }};
    self.order_.push_back(key);
    return obj;
  }
  // Destroys every singleton, newest first (called at interpreter exit).
  static void clear();
  template <typename T> static void erase() {
    SingletonManager &self = get_self();
    std::lock_guard<std::recursive_mutex> lock(self.mtx_);
    const std::type_index key(typeid(T));
    auto it = self.objects_.find(key);
    if (it == self.objects_.end())
      return;
    it->second.second(it->second.first);
    self.objects_.erase(it);
    for (auto o = self.order_.begin(); o != self.order_.end(); ++o)
      if (*o == key) {
        self.order_.erase(o);
        break;
      }
  }

private:
  static SingletonManager &get_self();
  std::recursive_mutex mtx_;
  std::unordered_map<std::type_index, std::pair<void *, std::function<void(void *)>>> objects_;
  vector<std::type_index> order_;
};

} // namespace nbla
#endif
