// C API over the nbla host layer for the Python front-end (ctypes): opaque handles for Variables and Functions,
// status codes plus a thread-local message instead of C++ exceptions.
#include <nbla/array/cpu_array.hpp>
#include <nbla/backend_registry.hpp>
#include <nbla/function/add2.hpp>
#include <nbla/function/div2.hpp>
#include <nbla/function/mul2.hpp>
#include <nbla/function/pow2.hpp>
#include <nbla/function/sub2.hpp>
#include <nbla/function/affine.hpp>
#include <nbla/function/binary_connect_affine.hpp>
#include <nbla/function/binary_connect_convolution.hpp>
#include <nbla/function/binary_weight_affine.hpp>
#include <nbla/function/binary_weight_convolution.hpp>
#include <nbla/function/concatenate.hpp>
#include <nbla/function/convolution.hpp>
#include <nbla/function/dequantize_linear.hpp>
#include <nbla/function/fixed_point_quantize.hpp>
#include <nbla/function/inq_affine.hpp>
#include <nbla/function/inq_convolution.hpp>
#include <nbla/function/min_max_quantize.hpp>
#include <nbla/function/pow2_quantize.hpp>
#include <nbla/function/prune.hpp>
#include <nbla/function/quantize_linear.hpp>
#include <nbla/function/relu.hpp>
#include <nbla/function/sink.hpp>
#include <nbla/hip/function/range_recorder.hpp>
#include <nbla/hip/init.hpp>
#include <nbla/init.hpp>

#include <cstring>

using namespace nbla;

namespace {

thread_local string g_error;
thread_local int g_error_code = 0;

template <typename F> int guarded(F &&f) {
  try {
    f();
    g_error_code = 0;
    return 0;
  } catch (const Exception &e) {
    g_error = e.what();
    g_error_code = (int)e.code() + 1;
  } catch (const std::exception &e) {
    g_error = e.what();
    g_error_code = (int)error_code::runtime + 1;
  } catch (...) {
    g_error = "unknown C++ exception";
    g_error_code = (int)error_code::unclassified + 1;
  }
  return g_error_code;
}

struct VarHandle {
  VariablePtr var;
};
struct FuncHandle {
  FunctionPtr func;
};

Variables to_variables(void **handles, int n) {
  Variables out;
  for (int i = 0; i < n; ++i)
    out.push_back(static_cast<VarHandle *>(handles[i])->var.get());
  return out;
}

NdArrayPtr pick(VarHandle *h, int which) { return which == 0 ? h->var->data() : h->var->grad(); }

Context cpu_ctx() { return Context({"cpu:float"}, "CpuCachedArray", "0"); }

vector<int> take_ints(const int64_t *&p, int n) {
  vector<int> out(p, p + n);
  p += n;
  return out;
}

FunctionPtr create_by_name(const string &name, const Context &ctx, const int64_t *ia, int ni, const double *fa, int nf,
                           const string &sarg) {
  auto need = [&](int want_i, int want_f) {
    NBLA_CHECK(ni >= want_i && nf >= want_f, error_code::value, "%s: expected at least %d integer and %d float arguments.",
               name.c_str(), want_i, want_f);
  };
  if (name == "FixedPointQuantize") {
    need(3, 1);
    return create_FixedPointQuantize(ctx, ia[0] != 0, (int)ia[1], (float)fa[0], ia[2] != 0);
  }
  if (name == "Pow2Quantize") {
    need(5, 0);
    return create_Pow2Quantize(ctx, ia[0] != 0, ia[1] != 0, (int)ia[2], (int)ia[3], ia[4] != 0);
  }
  if (name == "MinMaxQuantize") {
    need(3, 2);
    return create_MinMaxQuantize(ctx, (float)fa[0], ia[0] != 0, ia[1] != 0, ia[2] != 0, (float)fa[1]);
  }
  if (name == "BinaryWeightAffine") {
    need(1, 1);
    return create_BinaryWeightAffine(ctx, (int)ia[0], (float)fa[0]);
  }
  if (name == "BinaryConnectAffine") {
    need(1, 1);
    return create_BinaryConnectAffine(ctx, (int)ia[0], (float)fa[0]);
  }
  if (name == "BinaryWeightConvolution" || name == "BinaryConnectConvolution") {
    need(3, 1);
    const int64_t *p = ia;
    const int base_axis = (int)*p++, group = (int)*p++, nd = (int)*p++;
    NBLA_CHECK(ni >= 3 + 3 * nd, error_code::value, "%s: pad/stride/dilation arguments missing.", name.c_str());
    const vector<int> pad = take_ints(p, nd), stride = take_ints(p, nd), dilation = take_ints(p, nd);
    if (name == "BinaryWeightConvolution")
      return create_BinaryWeightConvolution(ctx, base_axis, pad, stride, dilation, group, (float)fa[0]);
    return create_BinaryConnectConvolution(ctx, base_axis, pad, stride, dilation, group, (float)fa[0]);
  }
  if (name == "INQAffine") {
    need(4, 0);
    const int64_t *p = ia;
    const int base_axis = (int)*p++, num_bits = (int)*p++, seed = (int)*p++, n_it = (int)*p++;
    NBLA_CHECK(ni >= 4 + n_it, error_code::value, "INQAffine: inq_iterations missing.");
    return create_INQAffine(ctx, base_axis, num_bits, take_ints(p, n_it), sarg, seed);
  }
  if (name == "INQConvolution") {
    need(5, 0);
    const int64_t *p = ia;
    const int base_axis = (int)*p++, group = (int)*p++, num_bits = (int)*p++, seed = (int)*p++, nd = (int)*p++;
    NBLA_CHECK(ni >= 6 + 3 * nd, error_code::value, "INQConvolution: pad/stride/dilation arguments missing.");
    const vector<int> pad = take_ints(p, nd), stride = take_ints(p, nd), dilation = take_ints(p, nd);
    const int n_it = (int)*p++;
    return create_INQConvolution(ctx, base_axis, pad, stride, dilation, group, num_bits, take_ints(p, n_it), sarg, seed);
  }
  if (name == "Affine") {
    need(1, 0);
    return create_Affine(ctx, (int)ia[0]);
  }
  if (name == "ReLU") {
    need(1, 0);
    return create_ReLU(ctx, ia[0] != 0);
  }
  if (name == "Add2") {
    need(1, 0);
    return create_Add2(ctx, ia[0] != 0);
  }
  if (name == "Sub2") {
    need(1, 0);
    return create_Sub2(ctx, ia[0] != 0);
  }
  if (name == "Mul2") {
    need(1, 0);
    return create_Mul2(ctx, ia[0] != 0);
  }
  if (name == "Div2") {
    need(1, 0);
    return create_Div2(ctx, ia[0] != 0);
  }
  if (name == "Pow2") {
    need(1, 0);
    return create_Pow2(ctx, ia[0] != 0);
  }
  if (name == "Concatenate") {
    need(1, 0);
    return create_Concatenate(ctx, (int)ia[0]);
  }
  if (name == "Convolution") {
    need(4, 0);
    const int64_t *p = ia;
    const int base_axis = (int)*p++, group = (int)*p++, channel_last = (int)*p++, nd = (int)*p++;
    NBLA_CHECK(ni >= 4 + 3 * nd, error_code::value, "Convolution: pad/stride/dilation arguments missing.");
    const vector<int> pad = take_ints(p, nd), stride = take_ints(p, nd), dilation = take_ints(p, nd);
    return create_Convolution(ctx, base_axis, pad, stride, dilation, group, channel_last != 0);
  }
  if (name == "QuantizeLinear") {
    need(2, 0);
    return create_QuantizeLinear(ctx, sarg, ia[0] != 0, (int)ia[1]);
  }
  if (name == "DequantizeLinear")
    return create_DequantizeLinear(ctx);
  if (name == "Prune") {
    need(0, 1);
    return create_Prune(ctx, (float)fa[0]);
  }
  if (name == "Sink") {
    need(1, 0);
    return create_Sink(ctx, ia[0] != 0);
  }
  if (name == "RangeRecorder") {
    need(2, 1);
    return create_RangeRecorder(ctx, (int)ia[0], fa[0], ia[1] != 0);
  }
  NBLA_ERROR(error_code::value, "Unknown function '%s'.", name.c_str());
}

int copy_string(const string &s, char *out, int n) {
  if (n <= 0)
    return (int)s.size();
  std::strncpy(out, s.c_str(), n - 1);
  out[n - 1] = '\0';
  return (int)s.size();
}

} // namespace

extern "C" {

NBLA_API const char *nblac_last_error() { return g_error.c_str(); }
// 0 = no error, else nbla::error_code + 1
NBLA_API int nblac_last_error_code() { return g_error_code; }

NBLA_API int nblac_init() {
  return guarded([] {
    init_cpu();
    init_hip();
  });
}

NBLA_API void nblac_shutdown() { SingletonManager::clear(); }

// ------------------------------------------------------------------ variables
NBLA_API void *nblac_variable_new(const int64_t *shape, int ndim) {
  VarHandle *h = nullptr;
  guarded([&] { h = new VarHandle{make_shared<Variable>(Shape_t(shape, shape + ndim))}; });
  return h;
}
NBLA_API void nblac_variable_free(void *v) { delete static_cast<VarHandle *>(v); }
NBLA_API int nblac_variable_ndim(void *v) { return (int)static_cast<VarHandle *>(v)->var->ndim(); }
NBLA_API void nblac_variable_shape(void *v, int64_t *out) {
  const Shape_t &s = static_cast<VarHandle *>(v)->var->shape();
  for (size_t i = 0; i < s.size(); ++i)
    out[i] = s[i];
}
NBLA_API int nblac_variable_reshape(void *v, const int64_t *shape, int ndim, int force) {
  return guarded([&] { static_cast<VarHandle *>(v)->var->reshape(Shape_t(shape, shape + ndim), force != 0); });
}
// Writes `size` host elements of `dtype` into data (which = 0) or grad (which = 1) through the host array class.
NBLA_API int nblac_variable_set(void *v, int which, const void *host, int dtype) {
  return guarded([&] {
    NdArrayPtr a = pick(static_cast<VarHandle *>(v), which);
    Array *arr = a->cast((dtypes)dtype, cpu_ctx(), true);
    std::memcpy(arr->pointer<void>(), host, (size_t)a->size() * sizeof_dtype((dtypes)dtype));
  });
}
// Reads through the host array class (a device-to-host synchronisation when the head lives on the device).
NBLA_API int nblac_variable_get(void *v, int which, void *host, int dtype) {
  return guarded([&] {
    NdArrayPtr a = pick(static_cast<VarHandle *>(v), which);
    const Array *arr = a->get((dtypes)dtype, cpu_ctx());
    std::memcpy(host, arr->const_pointer<void>(), (size_t)a->size() * sizeof_dtype((dtypes)dtype));
  });
}
NBLA_API int nblac_variable_fill(void *v, int which, double value) {
  return guarded([&] {
    NdArrayPtr a = pick(static_cast<VarHandle *>(v), which);
    if (value == 0.0)
      a->zero();
    else
      a->fill(value);
  });
}
// dtype of the head array, or -1 when nothing has been written yet.
NBLA_API int nblac_variable_dtype(void *v, int which) {
  int out = -1;
  guarded([&] { out = (int)pick(static_cast<VarHandle *>(v), which)->array()->dtype(); });
  return out;
}
NBLA_API int nblac_variable_head_array_class(void *v, int which, char *out, int n) {
  return copy_string(pick(static_cast<VarHandle *>(v), which)->array()->head_array_class(), out, n);
}
NBLA_API int64_t nblac_variable_modification_count(void *v, int which) {
  return (int64_t)pick(static_cast<VarHandle *>(v), which)->array()->modification_count();
}
// Device pointer of the data on the given hip device (synchronising it there); for tests and interop.
NBLA_API const void *nblac_variable_device_pointer(void *v, int which, int dtype, const char *device_id) {
  const void *p = nullptr;
  guarded([&] {
    Context ctx({"hip:float"}, "HipCachedArray", device_id);
    p = pick(static_cast<VarHandle *>(v), which)->get((dtypes)dtype, ctx)->const_pointer<void>();
  });
  return p;
}
// b becomes a view of a's data (and grad): same SyncedArrays, its own shape.
NBLA_API int nblac_variable_share(void *dst, void *src) {
  return guarded([&] {
    VarHandle *d = static_cast<VarHandle *>(dst), *s = static_cast<VarHandle *>(src);
    d->var->set_data(s->var->data()->view(d->var->shape()));
    d->var->set_grad(s->var->grad()->view(d->var->shape()));
  });
}

// dst's data (which = 0) or grad (which = 1) becomes a view of src's: `outputs=[param.data]` of the front-end.
NBLA_API int nblac_variable_share_array(void *dst, void *src, int which) {
  return guarded([&] {
    VarHandle *d = static_cast<VarHandle *>(dst), *s = static_cast<VarHandle *>(src);
    if (which == 0)
      d->var->set_data(s->var->data()->view(d->var->shape()));
    else
      d->var->set_grad(s->var->grad()->view(d->var->shape()));
  });
}

// ------------------------------------------------------------------ functions
NBLA_API void *nblac_function_create(const char *name, const char **backends, int n_backends, const char *array_class,
                                     const char *device_id, const int64_t *iargs, int ni, const double *fargs, int nf,
                                     const char *sarg) {
  FuncHandle *h = nullptr;
  guarded([&] {
    Context ctx(vector<string>(backends, backends + n_backends), array_class, device_id);
    h = new FuncHandle{create_by_name(name, ctx, iargs, ni, fargs, nf, sarg ? sarg : "")};
  });
  return h;
}
NBLA_API void nblac_function_free(void *f) { delete static_cast<FuncHandle *>(f); }
NBLA_API int nblac_function_name(void *f, char *out, int n) {
  return copy_string(static_cast<FuncHandle *>(f)->func->name(), out, n);
}
NBLA_API int nblac_function_min_outputs(void *f) { return static_cast<FuncHandle *>(f)->func->min_outputs(); }
NBLA_API int nblac_function_context(void *f, char *out, int n) {
  return copy_string(static_cast<FuncHandle *>(f)->func->context().to_string(), out, n);
}
NBLA_API int nblac_function_setup(void *f, void **inputs, int ni, void **outputs, int no) {
  return guarded([&] { static_cast<FuncHandle *>(f)->func->setup(to_variables(inputs, ni), to_variables(outputs, no)); });
}
NBLA_API int nblac_function_forward(void *f, void **inputs, int ni, void **outputs, int no) {
  return guarded(
      [&] { static_cast<FuncHandle *>(f)->func->forward(to_variables(inputs, ni), to_variables(outputs, no)); });
}
NBLA_API int nblac_function_recompute(void *f, void **inputs, int ni, void **outputs, int no) {
  return guarded(
      [&] { static_cast<FuncHandle *>(f)->func->recompute(to_variables(inputs, ni), to_variables(outputs, no)); });
}
NBLA_API int nblac_function_backward(void *f, void **inputs, int ni, void **outputs, int no) {
  return guarded([&] {
    static_cast<FuncHandle *>(f)->func->backward(to_variables(inputs, ni), to_variables(outputs, no),
                                                 vector<bool>(ni, true), vector<bool>(ni, false));
  });
}
// flags[i] bit 0: propagate_down, bit 1: accum, one byte per input
NBLA_API int nblac_function_backward_flags(void *f, void **inputs, int ni, void **outputs, int no,
                                           const unsigned char *flags) {
  return guarded([&] {
    vector<bool> prop(ni), accum(ni);
    for (int i = 0; i < ni; ++i) {
      prop[i] = flags[i] & 1;
      accum[i] = (flags[i] >> 1) & 1;
    }
    static_cast<FuncHandle *>(f)->func->backward(to_variables(inputs, ni), to_variables(outputs, no), prop, accum);
  });
}
NBLA_API void *nblac_function_copy(void *f) {
  FuncHandle *h = nullptr;
  guarded([&] { h = new FuncHandle{static_cast<FuncHandle *>(f)->func->copy()}; });
  return h;
}

// ------------------------------------------------------------- extension API
NBLA_API int nblac_hip_device_count() {
  int n = 0;
  guarded([&] { n = hip_get_device_count(); });
  return n;
}
NBLA_API int nblac_hip_device_synchronize(const char *device_id) {
  return guarded([&] { hip_device_synchronize(device_id); });
}
NBLA_API int nblac_hip_clear_memory_cache() {
  return guarded([&] { hip_clear_memory_cache(); });
}
// Comma separated list.
NBLA_API int nblac_array_classes(const char *backend, char *out, int n) {
  string joined;
  guarded([&] {
    init_cpu();
    init_hip();
    joined = string_join(string(backend) == "hip" ? hip_array_classes() : cpu_array_classes(), ",");
  });
  return copy_string(joined, out, n);
}
NBLA_API int64_t nblac_allocator_bytes(const char *backend, const char *device_id, int caching) {
  int64_t bytes = -1;
  guarded([&] {
    Context ctx({string(backend) + ":float"}, "", device_id);
    auto alloc = caching ? BackendUtils::caching_allocator(ctx) : BackendUtils::naive_allocator(ctx);
    bytes = (int64_t)alloc->get_total_allocated_bytes(device_id);
  });
  return bytes;
}

} // extern "C"
