// NdArray and Variable.
#include <nbla/variable.hpp>

namespace nbla {

NdArray::NdArray(const Shape_t &shape) : shape_(shape) {
  update_shape_info();
  array_ = make_shared<SyncedArray>(size_);
}
NdArray::NdArray(SyncedArrayPtr array, const Shape_t &shape) : array_(array), shape_(shape) {
  update_shape_info();
  NBLA_CHECK(array_->size() == size_, error_code::value, "Array size %ld does not match shape size %ld.",
             (long)array_->size(), (long)size_);
}
void NdArray::update_shape_info() {
  size_ = compute_size_by_shape(shape_);
  strides_ = get_c_contiguous_strides(shape_);
  ndim_ = (Size_t)shape_.size();
}
void NdArray::reshape(const Shape_t &shape, bool force) {
  if (shape_ == shape)
    return;
  const Size_t size = compute_size_by_shape(shape);
  if (size_ == size) {
    shape_ = shape;
    update_shape_info();
    return;
  }
  NBLA_CHECK(force, error_code::value, "Total dimensions not match. Set force=true if you want to resize array.");
  shape_ = shape;
  update_shape_info();
  array_ = make_shared<SyncedArray>(size_);
}
NdArray::Ptr NdArray::view(const Shape_t &shape) { return make_shared<NdArray>(array_, shape); }
Size_t NdArray::size(Size_t axis) const {
  if (axis <= 0)
    return size_;
  return compute_size_by_shape(shape_, (size_t)axis);
}
void NdArray::set_array(SyncedArrayPtr array) {
  NBLA_CHECK(size_ == array->size(), error_code::value, "Size must match.");
  array_ = array;
}

Variable::Variable(const Shape_t &shape) : shape_(shape) {
  update_shape_info();
  data_ = make_shared<NdArray>(shape_);
  grad_ = make_shared<NdArray>(shape_);
}
Variable::Variable(NdArrayPtr data) : shape_(data->shape()), data_(data) {
  update_shape_info();
  grad_ = make_shared<NdArray>(shape_);
}
void Variable::update_shape_info() {
  size_ = compute_size_by_shape(shape_);
  strides_ = get_c_contiguous_strides(shape_);
  ndim_ = (Size_t)shape_.size();
}
void Variable::reshape(const Shape_t &shape, bool force) {
  if (shape_ == shape)
    return;
  const Size_t size = compute_size_by_shape(shape);
  if (size_ == size) {
    shape_ = shape;
    update_shape_info();
    data_->reshape(shape, false);
    grad_->reshape(shape, false);
    return;
  }
  NBLA_CHECK(force, error_code::value, "Total dimensions not match. Set force=true if you want to resize array.");
  shape_ = shape;
  update_shape_info();
  data_->reshape(shape_, true);
  grad_->reshape(shape_, true);
}
Variable::Ptr Variable::view() {
  auto v = make_shared<Variable>(shape_);
  v->set_data(data_);
  v->set_grad(grad_);
  return v;
}
Variable::Ptr Variable::view(const Shape_t &shape) {
  NBLA_CHECK(compute_size_by_shape(shape) == size_, error_code::value, "The total size must be the same.");
  auto v = make_shared<Variable>(shape);
  v->set_data(data_->view(shape));
  v->set_grad(grad_->view(shape));
  return v;
}
Size_t Variable::size(Size_t axis) const {
  if (axis <= 0)
    return size_;
  return compute_size_by_shape(shape_, (size_t)axis);
}
void Variable::set_data(NdArrayPtr data) {
  NBLA_CHECK(data->shape() == shape_, error_code::value, "Shape must match.");
  data_ = data;
}
void Variable::set_grad(NdArrayPtr grad) {
  NBLA_CHECK(grad->shape() == shape_, error_code::value, "Shape must match.");
  grad_ = grad;
}

} // namespace nbla
