// SyncedArray: lazily materialised copies of one logical array, with head tracking.
#include <nbla/array_registry.hpp>
#include <nbla/synced_array.hpp>

namespace nbla {

namespace {
// One copy per device, array group and dtype.
string array_key(const Context &filtered, dtypes dtype) {
  return filtered.device_id + ":" + ArrayGroup::get_group(filtered.array_class) + ":" + dtype_to_string(dtype);
}
} // namespace

SyncedArray::SyncedArray(Size_t size) : size_(size) {
  head_.dtype = dtypes::FLOAT;
  zeroing_ = true; // a fresh array reads as zeros
}
SyncedArray::~SyncedArray() {}

dtypes SyncedArray::dtype() const {
  NBLA_CHECK(!head_.key.empty(), error_code::unclassified, "Array is not initialized.");
  return head_.dtype;
}

SyncedArray::ArrayDesc SyncedArray::sync(dtypes dtype, const Context &ctx_orig, bool write_only, int async_flags) {
  const Context ctx = ArrayCreator::filter_context(ctx_orig);
  ArrayDesc desc{array_key(ctx, dtype), ctx.array_class, dtype};
  const bool first = array_.empty();
  auto it = array_.find(desc.key);
  if (it == array_.end()) {
    ArrayPtr arr(ArrayCreator::create(size_, dtype, ctx));
    it = array_.insert({desc.key, {arr, false}}).first;
  } else {
    desc.array_class = it->second.first->context().array_class; // the class the copy was created with
  }
  if (first) {
    head_ = desc; // the first copy to exist is the head
    if (!zeroing_ && !filling_)
      it->second.second = true; // nothing to bring it up to date from: contents are whatever the memory holds
  }
  Array *arr = it->second.first.get();
  const bool up_to_date = it->second.second;
  if (write_only || size_ == 0) {
    it->second.second = true;
    return desc;
  }
  if (up_to_date)
    return desc;
  if (zeroing_) {
    arr->zero();
  } else if (filling_) {
    arr->fill(fill_value_);
  } else {
    auto head = array_.find(head_.key);
    NBLA_CHECK(head != array_.end() && head->second.second, error_code::unclassified,
               "SyncedArray has no valid head array to synchronise from.");
    Array *src = head->second.first.get();
    const string src_class = src->context().array_class;
    if (src_class == arr->context().array_class)
      arr->copy_from(src);
    else
      ArraySynchronizer::synchronize(src_class, src, arr->context().array_class, arr, async_flags);
  }
  it->second.second = true;
  return desc;
}

Array *SyncedArray::cast(dtypes dtype, const Context &ctx, bool write_only, int async_flags) {
  return cast_sp(dtype, ctx, write_only, async_flags).get();
}

ArrayPtr SyncedArray::cast_sp(dtypes dtype, const Context &ctx, bool write_only, int async_flags) {
  ArrayDesc desc = sync(dtype, ctx, write_only, async_flags);
  ArrayPtr keep = array_[desc.key].first;
  head_ = desc;
  // Everything else is stale once the head may be written.
  array_.clear();
  array_[desc.key] = {keep, true};
  clear_flags();
  modification_count_++;
  return keep;
}

const Array *SyncedArray::get(dtypes dtype, const Context &ctx, int async_flags) {
  return get_sp(dtype, ctx, async_flags).get();
}

ConstArrayPtr SyncedArray::get_sp(dtypes dtype, const Context &ctx, int async_flags) {
  ArrayDesc desc = sync(dtype, ctx, false, async_flags);
  return array_[desc.key].first;
}

const void *SyncedArray::data_ptr(dtypes dtype, const Context &ctx, bool write_only, int async_flags) {
  return cast_sp(dtype, ctx, write_only, async_flags)->const_pointer<void>();
}

void SyncedArray::zero() {
  clear_all_array();
  zeroing_ = true;
  filling_ = false;
  modification_count_++;
}

void SyncedArray::fill(float value) {
  clear_all_array();
  filling_ = true;
  zeroing_ = false;
  fill_value_ = value;
  modification_count_++;
}

void SyncedArray::copy_from(const SyncedArray *src) {
  NBLA_CHECK(src->size_ == size_, error_code::value, "Size mismatch.");
  SyncedArray *s = const_cast<SyncedArray *>(src);
  NBLA_CHECK(!s->head_.key.empty() || s->zeroing_ || s->filling_, error_code::value, "Source array is empty.");
  if (s->head_.key.empty()) { // nothing materialised yet: propagate the lazy state
    if (s->zeroing_)
      zero();
    else
      fill(s->fill_value_);
    return;
  }
  auto src_head = s->array_.find(s->head_.key);
  Context ctx = src_head->second.first->context();
  const Array *src_arr = s->get(s->head_.dtype, ctx);
  Array *dst_arr = cast(s->head_.dtype, ctx, true);
  dst_arr->copy_from(src_arr);
}

void SyncedArray::clear() {
  clear_all_array();
  clear_called_ = true;
}

void SyncedArray::clear_all_array() {
  array_.clear(); // head_ keeps the dtype readers expect; the lazy flags decide what the next copy holds
}

} // namespace nbla
