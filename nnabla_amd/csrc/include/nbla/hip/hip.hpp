// The hip backend singleton: array classes, allocators and synchronisation of MI355X devices
// (the counterpart of include/nbla/cpu.hpp for the "hip" backend name).
#ifndef NBLA_HIP_HPP_
#define NBLA_HIP_HPP_

#include <nbla/backend_base.hpp>
#include <nbla/singleton_manager.hpp>

namespace nbla {

class NBLA_API Hip : public BackendBase {
public:
  ~Hip();
  vector<string> array_classes() const override;
  void _set_array_classes(const vector<string> &a) override;
  void register_array_class(const string &name) override;
  shared_ptr<Allocator> caching_allocator() override;
  shared_ptr<Allocator> naive_allocator() override;
  void free_unused_host_caches() override;
  void device_synchronize(const string &device) override;
  void default_stream_synchronize(const string &device) override;
  void create_lms_streams(int device = -1) override;
  int get_device_count() const;

protected:
  vector<string> array_classes_;
  shared_ptr<Allocator> naive_allocator_, caching_allocator_;

private:
  friend SingletonManager;
  Hip();
};

} // namespace nbla
#endif
