// init_hip(): registers the hip backend, its array classes and synchronisers, and the "hip:float" implementations
// of the quantization functions in the nbla registries.
#include <nbla/array/cpu_array.hpp>
#include <nbla/array_registry.hpp>
#include <nbla/backend_registry.hpp>
#include <nbla/hip/array.hpp>
#include <nbla/hip/function/arithmetic.hpp>
#include <nbla/hip/function/binary.hpp>
#include <nbla/hip/function/inq.hpp>
#include <nbla/hip/function/quantize.hpp>
#include <nbla/hip/function/quantize_linear.hpp>
#include <nbla/hip/function/range_recorder.hpp>
#include <nbla/hip/init.hpp>
#include <nbla/init.hpp>

#include <mutex>

namespace nbla {

void init_hip() {
  static std::mutex mtx;
  static bool done = false;
  std::lock_guard<std::mutex> lock(mtx);
  if (done)
    return;
  done = true;
  init_cpu();

  NBLA_REGISTER_BACKEND("hip", []() { return SingletonManager::get<Hip>(); });

  // Entry 0 is the default array class of hip functions.
  NBLA_REGISTER_ARRAY_CREATOR(HipCachedArray);
  SingletonManager::get<Hip>()->register_array_class("HipCachedArray");
  NBLA_REGISTER_ARRAY_CREATOR(HipArray);
  SingletonManager::get<Hip>()->register_array_class("HipArray");
  NBLA_REGISTER_ARRAY_GROUP(HipArray, HipArray);
  NBLA_REGISTER_ARRAY_GROUP(HipCachedArray, HipArray);

  // Every pair SyncedArray can ask for: `.d` reads always go through a host array class.
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(HipArray, HipCachedArray, synchronizer_hip_array_hip_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(HipCachedArray, HipArray, synchronizer_hip_array_hip_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(HipArray, CpuArray, synchronizer_hip_array_cpu_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(HipArray, CpuCachedArray, synchronizer_hip_array_cpu_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(HipCachedArray, CpuArray, synchronizer_hip_array_cpu_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(HipCachedArray, CpuCachedArray, synchronizer_hip_array_cpu_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(CpuArray, HipArray, synchronizer_cpu_array_hip_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(CpuArray, HipCachedArray, synchronizer_cpu_array_hip_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(CpuCachedArray, HipArray, synchronizer_cpu_array_hip_array);
  NBLA_REGISTER_ARRAY_SYNCHRONIZER(CpuCachedArray, HipCachedArray, synchronizer_cpu_array_hip_array);

  // Function implementations, argument types as in the per-function registries.
  NBLA_REGISTER_FUNCTION_IMPL(FixedPointQuantize, FixedPointQuantizeHip<float>, "hip:float", bool, int, float, bool);
  NBLA_REGISTER_FUNCTION_IMPL(Pow2Quantize, Pow2QuantizeHip<float>, "hip:float", bool, bool, int, int, bool);
  NBLA_REGISTER_FUNCTION_IMPL(MinMaxQuantize, MinMaxQuantizeHip<float>, "hip:float", float, bool, bool, bool, float);
  NBLA_REGISTER_FUNCTION_IMPL(BinaryWeightAffine, BinaryWeightAffineHip<float>, "hip:float", int, float);
  NBLA_REGISTER_FUNCTION_IMPL(BinaryConnectAffine, BinaryConnectAffineHip<float>, "hip:float", int, float);
  NBLA_REGISTER_FUNCTION_IMPL(BinaryWeightConvolution, BinaryWeightConvolutionHip<float>, "hip:float", int,
                              const vector<int> &, const vector<int> &, const vector<int> &, int, float);
  NBLA_REGISTER_FUNCTION_IMPL(BinaryConnectConvolution, BinaryConnectConvolutionHip<float>, "hip:float", int,
                              const vector<int> &, const vector<int> &, const vector<int> &, int, float);
  typedef INQAffineHip<float, int> INQAffineHipFloatInt;
  NBLA_REGISTER_FUNCTION_IMPL(INQAffine, INQAffineHipFloatInt, "hip:float", int, int, const vector<int> &,
                              const string &, int);
  typedef INQConvolutionHip<float, int> INQConvolutionHipFloatInt;
  NBLA_REGISTER_FUNCTION_IMPL(INQConvolution, INQConvolutionHipFloatInt, "hip:float", int, const vector<int> &,
                              const vector<int> &, const vector<int> &, int, int, const vector<int> &, const string &,
                              int);
  NBLA_REGISTER_FUNCTION_IMPL(Affine, AffineHip<float>, "hip:float", int);
  NBLA_REGISTER_FUNCTION_IMPL(ReLU, ReLUHip<float>, "hip:float", bool);
  NBLA_REGISTER_FUNCTION_IMPL(Add2, Add2Hip<float>, "hip:float", bool);
  NBLA_REGISTER_FUNCTION_IMPL(Sub2, Sub2Hip<float>, "hip:float", bool);
  NBLA_REGISTER_FUNCTION_IMPL(Mul2, Mul2Hip<float>, "hip:float", bool);
  NBLA_REGISTER_FUNCTION_IMPL(Div2, Div2Hip<float>, "hip:float", bool);
  NBLA_REGISTER_FUNCTION_IMPL(Pow2, Pow2Hip<float>, "hip:float", bool);
  NBLA_REGISTER_FUNCTION_IMPL(Concatenate, ConcatenateHip<float>, "hip:float", int);
  NBLA_REGISTER_FUNCTION_IMPL(Convolution, ConvolutionHip<float>, "hip:float", int, const vector<int> &,
                              const vector<int> &, const vector<int> &, int, bool);
  NBLA_REGISTER_FUNCTION_IMPL(QuantizeLinear, QuantizeLinearHip<float>, "hip:float", const string &, bool, int);
  NBLA_REGISTER_FUNCTION_IMPL(DequantizeLinear, DequantizeLinearHip<float>, "hip:float");
  NBLA_REGISTER_FUNCTION_IMPL(Prune, PruneHip<float>, "hip:float", float);
  NBLA_REGISTER_FUNCTION_IMPL(Sink, SinkHip<float>, "hip:float", bool);
  NBLA_REGISTER_FUNCTION_IMPL(RangeRecorder, RangeRecorderHip<float>, "hip:float", int, double, bool);
}

} // namespace nbla
