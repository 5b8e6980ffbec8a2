// Library state: error reporting, per-device initialisation and the host-side
// calibration of the libm-dependent rounding cuts.
#include "common.hpp"

#include <cmath>
#include <cstdarg>
#include <cstring>
#include <mutex>

namespace nbla_hip {

namespace {

thread_local char g_error[512] = "";

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
bool g_calibrated = false;
bool g_device_ready[kMaxDevices] = {};
uint32_t g_host_tables[kNumCutTables][kNumBinades];
const uint32_t *g_device_tables[kMaxDevices] = {};

// One copy per device; written once by nbla_hip_init through its symbol address.
__device__ uint32_t d_cut_tables[kNumCutTables * kNumBinades];

inline float bits_to_float(uint32_t u) {
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// The three libm-dependent integer decisions, exactly as the reference writes them.

// pow2_quantize.cpp:60   roundf(log2f(a))
int step_pow2_round(float a) { return (int)std::round(std::log2(a)); }
// inq_affine.cpp:176-179  floorf(b) + (b - floorf(b) >= (float)log2(1.5))
int step_inq_exponent(float a) {
  const float b = std::log2(a);
  const float d = 0.58496250072115619;
  return (int)(std::floor(b) + (b - std::floor(b) >= d));
}
// inq_affine.cpp:161-164  same with the comparison against double log2(1.5)
int step_inq_n1(float a) {
  return (int)(std::floor(std::log2(a)) + (std::log2(a) - std::floor(std::log2(a)) >= std::log2(1.5)));
}

// Each decision f maps binade E to {E, E+1} and is a non-decreasing step in a,
// so one cut per binade describes it: f(u) = E + (u >= cut).  The cut is found
// by bisection over bit patterns (positive floats order like their bits) and
// the step shape is verified on both ends and on a window around the cut.
int calibrate(int (*f)(float), uint32_t *table, const char *name) {
  for (int idx = 0; idx < kNumBinades; ++idx) {
    const int E = idx - 149;
    const uint32_t lo = (idx < 23) ? (1u << idx) : ((uint32_t)(idx - 22) << 23);
    const uint32_t hi = (idx < 23) ? ((1u << (idx + 1)) - 1) : (lo | 0x7fffffu);
    const int flo = f(bits_to_float(lo)), fhi = f(bits_to_float(hi));
    if (flo != E || (fhi != E && fhi != E + 1))
      return fail(NBLA_HIP_ERR_RUNTIME, "%s calibration: binade 2^%d is not an {E,E+1} step (ends %d, %d)", name, E,
                  flo, fhi);
    uint32_t cut;
    if (fhi == E) {
      cut = hi + 1; // never reaches E+1 inside the binade
    } else {
      uint32_t a = lo, b = hi; // f(a) == E, f(b) == E+1
      while (b - a > 1) {
        const uint32_t mid = a + (b - a) / 2;
        if (f(bits_to_float(mid)) > E)
          b = mid;
        else
          a = mid;
      }
      cut = b;
    }
    const uint32_t w0 = (cut - lo > 192) ? cut - 192 : lo;
    const uint32_t w1 = (hi - cut > 192 && cut <= hi) ? cut + 192 : hi;
    for (uint32_t u = w0; u <= w1; ++u) {
      const int want = E + (u >= cut ? 1 : 0);
      if (f(bits_to_float(u)) != want)
        return fail(NBLA_HIP_ERR_RUNTIME, "%s calibration: host libm is not monotone near 0x%08x", name, u);
    }
    table[idx] = cut;
  }
  return NBLA_HIP_OK;
}

} // namespace

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int fail_hip(hipError_t err, const char *what) {
  snprintf(g_error, sizeof(g_error), "%s: %s (%s)", what, hipGetErrorString(err), hipGetErrorName(err));
  return (int)err;
}

const uint32_t *device_cut_table(int which) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices || !g_device_tables[dev])
    return nullptr;
  return g_device_tables[dev] + which * kNumBinades;
}

int ensure_init() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return fail_hip(e, "hipGetDevice");
  if (dev >= 0 && dev < kMaxDevices && g_device_ready[dev])
    return NBLA_HIP_OK;
  return nbla_hip_init(dev);
}

} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

int nbla_hip_init(int device) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (device < 0 || device >= kMaxDevices)
    return fail(NBLA_HIP_ERR_VALUE, "device index %d out of range", device);
  hipError_t e = hipSetDevice(device);
  if (e != hipSuccess)
    return fail_hip(e, "hipSetDevice");
  if (g_device_ready[device])
    return NBLA_HIP_OK;
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess)
    return fail_hip(e, "hipGetDeviceProperties");
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(NBLA_HIP_ERR_RUNTIME, "device %d is %s; this library is built for gfx950 only", device,
                prop.gcnArchName);
  if (!g_calibrated) {
    int rc = calibrate(step_pow2_round, g_host_tables[kCutPow2Round], "roundf(log2f)");
    if (rc)
      return rc;
    rc = calibrate(step_inq_exponent, g_host_tables[kCutInqExponent], "INQ exponent");
    if (rc)
      return rc;
    rc = calibrate(step_inq_n1, g_host_tables[kCutInqN1], "INQ n1");
    if (rc)
      return rc;
    g_calibrated = true;
  }
  void *sym = nullptr;
  e = hipGetSymbolAddress(&sym, HIP_SYMBOL(d_cut_tables));
  if (e != hipSuccess)
    return fail_hip(e, "hipGetSymbolAddress(cut tables)");
  e = hipMemcpy(sym, g_host_tables, sizeof(g_host_tables), hipMemcpyHostToDevice);
  if (e != hipSuccess)
    return fail_hip(e, "hipMemcpy(cut tables)");
  g_device_tables[device] = static_cast<const uint32_t *>(sym);
  const int rc_scratch = register_static_scratch(device);
  if (rc_scratch)
    return rc_scratch;
  g_device_ready[device] = true;
  return NBLA_HIP_OK;
}

const char *nbla_hip_last_error(void) { return g_error; }

const char *nbla_hip_version(void) { return "nbla_hip_kernels 0.1 (gfx950)"; }

int nbla_hip_cut_table(int which, uint32_t *out277) {
  if (which < 0 || which >= kNumCutTables || !out277)
    return fail(NBLA_HIP_ERR_VALUE, "cut table index %d out of range", which);
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_calibrated) {
      int rc = calibrate(step_pow2_round, g_host_tables[kCutPow2Round], "roundf(log2f)");
      if (!rc)
        rc = calibrate(step_inq_exponent, g_host_tables[kCutInqExponent], "INQ exponent");
      if (!rc)
        rc = calibrate(step_inq_n1, g_host_tables[kCutInqN1], "INQ n1");
      if (rc)
        return rc;
      g_calibrated = true;
    }
  }
  std::memcpy(out277, g_host_tables[which], sizeof(uint32_t) * kNumBinades);
  return NBLA_HIP_OK;
}

} // extern "C"
