// The host backend singleton (mirrors include/nbla/cpu.hpp, src/nbla/cpu.cpp).
#ifndef NBLA_CPU_HPP_
#define NBLA_CPU_HPP_

#include <nbla/backend_base.hpp>
#include <nbla/singleton_manager.hpp>

namespace nbla {

class NBLA_API Cpu : public BackendBase {
public:
  ~Cpu();
  vector<string> array_classes() const override;
  void _set_array_classes(const vector<string> &a) override;
  void register_array_class(const string &name) override;
  shared_ptr<Allocator> caching_allocator() override;
  shared_ptr<Allocator> naive_allocator() override;
  void free_unused_host_caches() override;
  void device_synchronize(const string &device) override;
  void default_stream_synchronize(const string &device) override;
  void create_lms_streams(int device = -1) override;

protected:
  vector<string> array_classes_;
  shared_ptr<Allocator> naive_allocator_, caching_allocator_;

private:
  friend SingletonManager;
  Cpu();
};

} // namespace nbla
#endif
