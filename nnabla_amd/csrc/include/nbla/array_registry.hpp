// Registries that let SyncedArray create arrays of any class and move data between
// classes (mirrors include/nbla/array_registry.hpp:33-137).
#ifndef NBLA_ARRAY_REGISTRY_HPP_
#define NBLA_ARRAY_REGISTRY_HPP_

#include <nbla/array.hpp>

#include <functional>
#include <map>

namespace nbla {

class NBLA_API ArrayCreator {
public:
  typedef std::function<Array *(const Size_t, dtypes, const Context &, const AllocatorMemoryPtr, const Size_t)> Creator;
  typedef std::function<Context(const Context &)> FilterContext;
  static Array *create(const Size_t size, dtypes dtype, const Context &ctx, const AllocatorMemoryPtr mem = nullptr,
                       const Size_t offset = 0);
  static Context filter_context(const Context &ctx);
  static void add_creator(const string &name, Creator creator, FilterContext filter_context);
  static vector<string> get_array_classes();

private:
  static std::map<string, std::pair<Creator, FilterContext>> &registry();
};

class NBLA_API ArraySynchronizer {
public:
  typedef std::function<void(Array *, Array *, int)> Synchronizer;
  static void synchronize(const string &src_class, Array *src_array, const string &dst_class, Array *dst_array,
                          int async_flags = 0);
  static void add_synchronizer(const string &src_class, const string &dst_class, Synchronizer synchronizer);

private:
  static std::map<std::pair<string, string>, Synchronizer> &registry();
};

// Array classes of one group share storage semantics (e.g. cached/uncached variants on one device), so a
// SyncedArray keeps a single array per (device, group, dtype).
class NBLA_API ArrayGroup {
public:
  static void add_group(const string &array_class, const string &group_name);
  static string get_group(const string &array_class);

private:
  static std::map<string, string> &registry();
};

#define NBLA_REGISTER_ARRAY_CREATOR(CLS)                                                                               \
  ::nbla::ArrayCreator::add_creator(                                                                                   \
      #CLS,                                                                                                            \
      [](const ::nbla::Size_t size, ::nbla::dtypes dtype, const ::nbla::Context &ctx,                                  \
         const ::nbla::AllocatorMemoryPtr mem, const ::nbla::Size_t offset) -> ::nbla::Array * {                       \
        return new CLS(size, dtype, ctx, mem, offset);                                                                 \
      },                                                                                                               \
      CLS::filter_context)
#define NBLA_REGISTER_ARRAY_SYNCHRONIZER(SRC_CLASS, DST_CLASS, SYNCHRONIZER)                                           \
  ::nbla::ArraySynchronizer::add_synchronizer(#SRC_CLASS, #DST_CLASS, SYNCHRONIZER)
#define NBLA_REGISTER_ARRAY_GROUP(CLS, GROUP) ::nbla::ArrayGroup::add_group(#CLS, #GROUP)

} // namespace nbla
#endif
