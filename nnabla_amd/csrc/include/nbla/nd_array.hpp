// Shape + SyncedArray (mirrors include/nbla/nd_array.hpp).
#ifndef NBLA_ND_ARRAY_HPP_
#define NBLA_ND_ARRAY_HPP_

#include <nbla/synced_array.hpp>

namespace nbla {

class NBLA_API NdArray {
  SyncedArrayPtr array_;
  Shape_t shape_, strides_;
  Size_t size_, ndim_;
  void update_shape_info();

public:
  typedef shared_ptr<NdArray> Ptr;
  template <typename... Args> static Ptr create(Args... args) { return make_shared<NdArray>(args...); }
  explicit NdArray(const Shape_t &shape = {});
  NdArray(SyncedArrayPtr array, const Shape_t &shape);
  // force: replace the underlying array when the element count changes.
  void reshape(const Shape_t &shape, bool force = false);
  Ptr view(const Shape_t &shape);
  const Shape_t &shape() const { return shape_; }
  const Shape_t &strides() const { return strides_; }
  Size_t size(Size_t axis = -1) const;
  Size_t ndim() const { return ndim_; }
  SyncedArrayPtr array() { return array_; }
  void set_array(SyncedArrayPtr array);
  void zero() { array_->zero(); }
  void fill(double v) { array_->fill((float)v); }
  const Array *get(dtypes dtype, const Context &ctx) { return array_->get(dtype, ctx); }
  ConstArrayPtr get_sp(dtypes dtype, const Context &ctx) { return array_->get_sp(dtype, ctx); }
  Array *cast(dtypes dtype, const Context &ctx, bool write_only = false) { return array_->cast(dtype, ctx, write_only); }
  ArrayPtr cast_sp(dtypes dtype, const Context &ctx, bool write_only = false) {
    return array_->cast_sp(dtype, ctx, write_only);
  }
};
typedef NdArray::Ptr NdArrayPtr;

} // namespace nbla
#endif
