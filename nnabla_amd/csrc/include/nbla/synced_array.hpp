// A logical array that is materialised lazily per (device, array group, dtype) and keeps track of which copy is
// current (mirrors include/nbla/synced_array.hpp and the semantics of src/nbla/synced_array.cpp).
#ifndef NBLA_SYNCED_ARRAY_HPP_
#define NBLA_SYNCED_ARRAY_HPP_

#include <nbla/array.hpp>

#include <map>

namespace nbla {

class NBLA_API SyncedArray : public std::enable_shared_from_this<SyncedArray> {
  struct ArrayDesc {
    string key;
    string array_class;
    dtypes dtype;
  };
  ArrayDesc head_;
  bool zeroing_ = false;
  bool filling_ = false;
  float fill_value_ = 0.0f;
  Size_t size_;
  std::map<string, std::pair<ArrayPtr, bool>> array_; // key -> (array, is up to date)
  size_t modification_count_ = 0;
  bool clear_called_ = false;

public:
  explicit SyncedArray(Size_t size);
  ~SyncedArray();
  SyncedArray(const SyncedArray &) = delete;
  SyncedArray &operator=(const SyncedArray &) = delete;

  // Read/write access: the returned array becomes the only current copy.  write_only skips bringing it up to date.
  Array *cast(dtypes dtype, const Context &ctx, bool write_only = false, int async_flags = 0);
  ArrayPtr cast_sp(dtypes dtype, const Context &ctx, bool write_only = false, int async_flags = 0);
  // Read access: the returned array is brought up to date; the head stays where it was.
  const Array *get(dtypes dtype, const Context &ctx, int async_flags = 0);
  ConstArrayPtr get_sp(dtypes dtype, const Context &ctx, int async_flags = 0);
  // Raw pointer of the current head array without any synchronisation (nullptr before the first write).
  const void *data_ptr(dtypes dtype, const Context &ctx, bool write_only = false, int async_flags = 0);

  dtypes dtype() const;
  string head_array_class() const { return head_.array_class; }
  size_t get_num_arrays() const { return array_.size(); }
  Size_t size() const { return size_; }
  // Lazily evaluated: executed on whichever array is requested next.
  void zero();
  void fill(float value);
  bool zeroing() const { return zeroing_; }
  size_t modification_count() const { return modification_count_; }
  bool clear_called() const { return clear_called_; }
  void copy_from(const SyncedArray *src);
  void clear();

private:
  ArrayDesc sync(dtypes dtype, const Context &ctx, bool write_only, int async_flags);
  void clear_all_array();
  void clear_flags() { zeroing_ = filling_ = false; }
};
typedef shared_ptr<SyncedArray> SyncedArrayPtr;

} // namespace nbla
#endif
