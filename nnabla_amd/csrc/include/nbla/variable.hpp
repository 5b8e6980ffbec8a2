// data + grad NdArrays sharing one shape (mirrors include/nbla/variable.hpp).
#ifndef NBLA_VARIABLE_HPP_
#define NBLA_VARIABLE_HPP_

#include <nbla/nd_array.hpp>

namespace nbla {

class NBLA_API Variable {
  Shape_t shape_, strides_;
  Size_t size_, ndim_;
  NdArrayPtr data_, grad_;
  void update_shape_info();

public:
  typedef shared_ptr<Variable> Ptr;
  template <typename... Args> static Ptr create(Args... args) { return make_shared<Variable>(args...); }
  explicit Variable(const Shape_t &shape = {});
  explicit Variable(NdArrayPtr data);
  void reshape(const Shape_t &shape, bool force);
  Ptr view();
  Ptr view(const Shape_t &shape);
  const Shape_t &shape() const { return shape_; }
  const Shape_t &strides() const { return strides_; }
  Size_t size(Size_t axis = -1) const;
  Size_t ndim() const { return ndim_; }
  NdArrayPtr data() { return data_; }
  NdArrayPtr grad() { return grad_; }
  void set_data(NdArrayPtr data);
  void set_grad(NdArrayPtr grad);

  template <typename T> const T *get_data_pointer(const Context &ctx) {
    return data_->get(get_dtype<T>(), ctx)->template const_pointer<T>();
  }
  template <typename T> const T *get_grad_pointer(const Context &ctx) {
    return grad_->get(get_dtype<T>(), ctx)->template const_pointer<T>();
  }
  template <typename T> T *cast_data_and_get_pointer(const Context &ctx, bool write_only = false) {
    return data_->cast(get_dtype<T>(), ctx, write_only)->template pointer<T>();
  }
  template <typename T> T *cast_grad_and_get_pointer(const Context &ctx, bool write_only = false) {
    return grad_->cast(get_dtype<T>(), ctx, write_only)->template pointer<T>();
  }
};
typedef Variable::Ptr VariablePtr;
typedef vector<Variable *> Variables;

} // namespace nbla
#endif
