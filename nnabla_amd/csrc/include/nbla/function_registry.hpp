// Per-function registries keyed by backend string with ordered fallback over Context::backend
// (mirrors include/nbla/function_registry.hpp:57-197).
#ifndef NBLA_FUNCTION_REGISTRY_HPP_
#define NBLA_FUNCTION_REGISTRY_HPP_

#include <nbla/function.hpp>
#include <nbla/init.hpp>

#include <functional>
#include <mutex>

namespace nbla {

template <typename Item> class FunctionDbItem;

template <typename Base, typename... Args> struct FunctionDbItem<Base(Args...)> {
  typedef std::function<shared_ptr<Base>(const Context &ctx, Args...)> function_t;
  string backend;
  function_t function;
};

// The database of one Function: a list of (backend, creator).
template <typename Item> class FunctionDb {
  vector<shared_ptr<Item>> items_;

public:
  // The creator of the first entry of `backend` (in the context's order) that has an implementation.
  typename Item::function_t query(const vector<string> &backend) {
    for (const string &b : backend)
      for (auto &item : items_)
        if (item->backend == b)
          return item->function;
    vector<string> have;
    for (auto &item : items_)
      have.push_back(item->backend);
    NBLA_ERROR(error_code::value, "Any of [%s] could not be found in [%s]", string_join(backend, ", ").c_str(),
               string_join(have, ", ").c_str());
  }
  void add(shared_ptr<Item> item) { items_.push_back(item); }
  vector<string> backends() const {
    vector<string> out;
    for (auto &item : items_)
      out.push_back(item->backend);
    return out;
  }
};

template <typename Base, typename... Args> class FunctionRegistry {
public:
  typedef FunctionDbItem<Base(Args...)> item_t;
  FunctionDb<item_t> function_db_;
  std::mutex mtx_;
  shared_ptr<Base> create(const Context &ctx, Args... args) {
    typename item_t::function_t f;
    {
      std::lock_guard<std::mutex> lock(mtx_);
      f = function_db_.query(ctx.backend);
    }
    return f(ctx, args...);
  }
  void add(shared_ptr<item_t> item) {
    std::lock_guard<std::mutex> lock(mtx_);
    function_db_.add(item);
  }
};

// In the function's header.
#define NBLA_REGISTER_FUNCTION_HEADER(NAME, ...)                                                                       \
  NBLA_API ::nbla::FunctionRegistry<::nbla::Function, ##__VA_ARGS__> &get_##NAME##Registry();                          \
  template <typename... CreateArgs__>                                                                                  \
  inline ::nbla::shared_ptr<::nbla::Function> create_##NAME(const ::nbla::Context &ctx, CreateArgs__ &&... args) {     \
    ::nbla::init_cpu();                                                                                                \
    return get_##NAME##Registry().create(ctx, std::forward<CreateArgs__>(args)...);                                    \
  }

// In exactly one source file of the core.
#define NBLA_REGISTER_FUNCTION_SOURCE(NAME, ...)                                                                       \
  ::nbla::FunctionRegistry<::nbla::Function, ##__VA_ARGS__> &get_##NAME##Registry() {                                  \
    static ::nbla::FunctionRegistry<::nbla::Function, ##__VA_ARGS__> registry;                                         \
    return registry;                                                                                                   \
  }

// In a backend's init_<ext>(): adds implementation CLS under BACKEND.
#define NBLA_REGISTER_FUNCTION_IMPL(BASE, CLS, BACKEND, ...)                                                           \
  {                                                                                                                    \
    typedef ::nbla::FunctionDbItem<::nbla::Function(__VA_ARGS__)> item_t__;                                            \
    auto item__ = ::nbla::make_shared<item_t__>();                                                                     \
    item__->backend = BACKEND;                                                                                         \
    item__->function = ::nbla::detail::creator_of<CLS, ##__VA_ARGS__>();                                               \
    get_##BASE##Registry().add(item__);                                                                                \
  }

namespace detail {
template <typename CLS, typename... Args>
std::function<shared_ptr<Function>(const Context &, Args...)> creator_of() {
  return [](const Context &ctx, Args... args) -> shared_ptr<Function> { return make_shared<CLS>(ctx, args...); };
}
} // namespace detail

} // namespace nbla
#endif
