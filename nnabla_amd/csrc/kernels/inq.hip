// Incremental Network Quantization (INQAffine / INQConvolution): the weight
// logic of the forward pass on the device -- restore fixed weights, select the
// weights to fix, quantize fixed weights to signed powers of two, snapshot --
// followed by the fp32-faithful product on the matrix cores.
//
// The two libm-dependent decisions of the reference (the exponent of a weight,
// inq_affine.cpp:176-179, and n1 from max|w|, :161-164) are taken from per-binade
// cut tables calibrated against the host's log2f when the library initialises.
#include "common.hpp"
#include "conv_geom.hpp"
#include "gemm_layout.hpp"
#include "internal.hpp"

#include <cstring> // rocprim's texture iterator calls memset without including it
#include <rocprim/rocprim.hpp>

#include <cmath>
#include <vector>

namespace nbla_hip {
namespace {

constexpr int kBlk = 256;
constexpr int kMaxPartials = 1024;

struct InqParams {
  int n1, n2;
  float thr;
  int pad;
};

struct InqWorkspace {
  size_t params_off, partial_off, keys_in_off, keys_out_off, vals_in_off, vals_out_off, scan_off, temp_off, temp_bytes,
      draws_off, total;
};

size_t rocprim_temp_bytes(int64_t size) {
  size_t sort_bytes = 0, scan_bytes = 0;
  uint32_t *k = nullptr;
  int *f = nullptr;
  (void)rocprim::radix_sort_pairs_desc(nullptr, sort_bytes, k, k, k, k, (size_t)size, 0, 32, (hipStream_t)0);
  (void)rocprim::inclusive_scan(nullptr, scan_bytes, f, f, (size_t)size, rocprim::plus<int>(), (hipStream_t)0);
  return sort_bytes > scan_bytes ? sort_bytes : scan_bytes;
}

InqWorkspace plan_inq(int64_t size, int selection) {
  InqWorkspace w;
  size_t off = 0;
  w.params_off = off;
  off += 256;
  w.partial_off = off;
  off += round_up(kMaxPartials * sizeof(uint32_t), 256);
  const size_t arr = round_up((size_t)size * 4, 256);
  w.keys_in_off = w.keys_out_off = w.vals_in_off = w.vals_out_off = w.scan_off = w.temp_off = w.draws_off = off;
  w.temp_bytes = 0;
  if (selection == 1) { // largest_abs: sort pairs + scan
    w.keys_in_off = off, off += arr;
    w.keys_out_off = off, off += arr;
    w.vals_in_off = off, off += arr;
    w.vals_out_off = off, off += arr;
    w.scan_off = off, off += arr;
    w.temp_bytes = round_up(rocprim_temp_bytes(size), 256);
    w.temp_off = off, off += w.temp_bytes;
  } else if (selection == 2) { // random: scan + uploaded draws
    w.keys_in_off = off, off += arr; // learnable flags
    w.scan_off = off, off += arr;
    w.temp_bytes = round_up(rocprim_temp_bytes(size), 256);
    w.temp_off = off, off += w.temp_bytes;
    w.draws_off = off, off += round_up((size_t)size, 256);
  }
  w.total = off;
  return w;
}

// Step A (inq_affine.cpp:95-102) fused with the max|w| scan of step C (:153-158).
__global__ __launch_bounds__(kBlk) void inq_restore_absmax(float *__restrict__ W, const float *__restrict__ old_W,
                                                           const int *__restrict__ old_I, int64_t size, int vec,
                                                           uint32_t *__restrict__ partial) {
  typedef float f4_t __attribute__((ext_vector_type(4)));
  typedef int i4_t __attribute__((ext_vector_type(4)));
  uint32_t mx = 0u; // bits of a non-negative float order like the float
  auto take = [&](float w) {
    const uint32_t u = __float_as_uint(w) & 0x7fffffffu;
    if (u <= 0x7f800000u && u > mx) // NaN never compares greater
      mx = u;
  };
  const int64_t stride = (int64_t)gridDim.x * kBlk;
  int64_t done = 0;
  if (vec) { // 16-byte aligned arrays: four weights per lane and access, two accesses in flight
    const int64_t n4 = size / 4;
    for (int64_t i = (int64_t)blockIdx.x * kBlk + threadIdx.x; i < n4; i += 2 * stride) {
      const int64_t j = i + stride;
      const bool second = j < n4;
      // the indicators first: a quad whose four weights are all fixed is taken from the snapshot without reading W
      const i4_t f0 = reinterpret_cast<const i4_t *>(old_I)[i];
      const i4_t f1 = second ? reinterpret_cast<const i4_t *>(old_I)[j] : f0;
      const bool all0 = f0.x == 1 && f0.y == 1 && f0.z == 1 && f0.w == 1;
      const bool any0 = f0.x == 1 || f0.y == 1 || f0.z == 1 || f0.w == 1;
      const bool all1 = f1.x == 1 && f1.y == 1 && f1.z == 1 && f1.w == 1;
      const bool any1 = f1.x == 1 || f1.y == 1 || f1.z == 1 || f1.w == 1;
      f4_t w0 = {0.0f, 0.0f, 0.0f, 0.0f}, w1 = w0, o0 = w0, o1 = w0;
      if (!all0)
        w0 = reinterpret_cast<const f4_t *>(W)[i];
      if (any0)
        o0 = reinterpret_cast<const f4_t *>(old_W)[i];
      if (second && !all1)
        w1 = reinterpret_cast<const f4_t *>(W)[j];
      if (second && any1)
        o1 = reinterpret_cast<const f4_t *>(old_W)[j];
      if (any0) {
        w0.x = f0.x == 1 ? o0.x : w0.x, w0.y = f0.y == 1 ? o0.y : w0.y;
        w0.z = f0.z == 1 ? o0.z : w0.z, w0.w = f0.w == 1 ? o0.w : w0.w;
        reinterpret_cast<f4_t *>(W)[i] = w0;
      }
      take(w0.x), take(w0.y), take(w0.z), take(w0.w);
      if (second) {
        if (any1) {
          w1.x = f1.x == 1 ? o1.x : w1.x, w1.y = f1.y == 1 ? o1.y : w1.y;
          w1.z = f1.z == 1 ? o1.z : w1.z, w1.w = f1.w == 1 ? o1.w : w1.w;
          reinterpret_cast<f4_t *>(W)[j] = w1;
        }
        take(w1.x), take(w1.y), take(w1.z), take(w1.w);
      }
    }
    done = n4 * 4;
  }
  for (int64_t i = done + (int64_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += stride) {
    float w = W[i];
    if (old_I[i] == 1) {
      w = old_W[i];
      W[i] = w;
    }
    take(w);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const uint32_t o = __shfl_xor(mx, off);
    mx = o > mx ? o : mx;
  }
  __shared__ uint32_t s_mx[kBlk / 64];
  if ((threadIdx.x & 63) == 0)
    s_mx[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kBlk / 64; ++w)
      mx = s_mx[w] > mx ? s_mx[w] : mx;
    partial[blockIdx.x] = mx;
  }
}

// n1, n2 and the pruning threshold (inq_affine.cpp:157-166).  `levels` is the
// host's (int)pow(2, num_bits - 2).
__global__ __launch_bounds__(64) void inq_finalize(const uint32_t *__restrict__ partial, int nparts, int levels,
                                                   const uint32_t *__restrict__ n1_cuts, InqParams *__restrict__ params,
                                                   ColumnScratch cols) {
  // the column statistics that the quantize pass will gather (cols.cmax null: none wanted) start from their neutral
  // values
  if (cols.cmax) {
    for (int64_t i = threadIdx.x; i < cols.rows; i += 64) {
      cols.cmax[i] = 0u;
      cols.cmin[i] = 0xffffffffu;
    }
    if (threadIdx.x == 0)
      *cols.flag = 0;
  }
  uint32_t mx = 0u;
  for (int i = threadIdx.x; i < nparts; i += 64)
    mx = partial[i] > mx ? partial[i] : mx;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const uint32_t o = __shfl_xor(mx, off);
    mx = o > mx ? o : mx;
  }
  if (threadIdx.x != 0)
    return;
  if (mx == 0u)
    mx = 0x3f800000u; // max_absval == 0 -> 1
  int n1;
  if (mx >= 0x7f800000u) {
    n1 = 128; // infinite weight: the reference's int conversion is undefined here
  } else {
    const int idx = binade_of(mx);
    n1 = binade_exponent(idx) + (mx >= n1_cuts[idx] ? 1 : 0);
  }
  const int n2 = n1 + 1 - levels;
  const int te = n2 - 1;
  float thr;
  if (te > 127)
    thr = __uint_as_float(0x7f800000u);
  else if (te < -149)
    thr = 0.0f;
  else
    thr = pow2_int(te);
  InqParams p;
  p.n1 = n1;
  p.n2 = n2;
  p.thr = thr;
  p.pad = 0;
  *params = p;
}

// Step C for one fixed weight (:168-190).
__device__ __forceinline__ float inq_quantize_value(float w, const InqParams &p, const uint32_t *s_cut) {
  const uint32_t u = __float_as_uint(w) & 0x7fffffffu;
  const float a = __uint_as_float(u);
  if (a < p.thr)
    return 0.0f;
  if (u < 0x7f800000u && u != 0u) {
    const int idx = binade_of(u);
    int e = binade_exponent(idx) + (u >= s_cut[idx] ? 1 : 0);
    if (e > p.n1)
      e = p.n1;
    if (e < p.n2)
      e = p.n2;
    float q;
    if (e > 127)
      q = __uint_as_float(0x7f800000u);
    else if (e < -149)
      q = 0.0f;
    else
      q = pow2_int(e);
    return (w < 0.0f) ? -q : q;
  }
  // zero with a zero threshold, infinities and NaN: outside the reference's defined behaviour; left as they are
  return w;
}

// Step C for the fixed weights (:168-190) and step F (:203-204).
__global__ __launch_bounds__(kBlk) void inq_quantize(float *__restrict__ W, int *__restrict__ I, float *__restrict__ old_W,
                                                     int *__restrict__ old_I, int64_t size, int fix_all,
                                                     const InqParams *__restrict__ params,
                                                     const uint32_t *__restrict__ e_cuts) {
  __shared__ uint32_t s_cut[kNumBinades];
  for (int i = threadIdx.x; i < kNumBinades; i += kBlk)
    s_cut[i] = e_cuts[i];
  __syncthreads();
  const InqParams p = *params;
  for (int64_t i = (int64_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (int64_t)gridDim.x * kBlk) {
    float w = W[i];
    const int ind = fix_all ? 1 : I[i];
    if (ind == 1)
      w = inq_quantize_value(w, p, s_cut);
    W[i] = w;
    if (fix_all)
      I[i] = ind; // otherwise unchanged
    old_W[i] = w;
    old_I[i] = ind;
  }
}

// The same for a weight matrix [R, C] (C % 4 == 0, 16-byte aligned) that is about to become the column-scaled digit
// operand of the product: the pass also gathers that operand's column statistics (largest / smallest non-zero
// magnitude per column, the flag for elements that are neither zero nor a normal power of two) from the values it
// writes, so the operand needs no pass of its own over W for them.  Block = 64 column quads x 4 row groups over a
// slab of rows, as in the stand-alone statistics kernel.
__global__ __launch_bounds__(kBlk) void inq_quantize_columns(float *__restrict__ W, int *__restrict__ I,
                                                             float *__restrict__ old_W, int *__restrict__ old_I,
                                                             int64_t R, int64_t C, int slab, int fix_all,
                                                             const InqParams *__restrict__ params,
                                                             const uint32_t *__restrict__ e_cuts, ColumnScratch cols) {
  typedef float f4_t __attribute__((ext_vector_type(4)));
  typedef int i4_t __attribute__((ext_vector_type(4)));
  static_assert(kBlk == 256, "64 column quads x 4 row groups");
  __shared__ uint32_t s_cut[kNumBinades];
  __shared__ uint32_t part[4][256], part_min[4][256];
  for (int i = threadIdx.x; i < kNumBinades; i += kBlk)
    s_cut[i] = e_cuts[i];
  __syncthreads();
  const InqParams p = *params;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int64_t c0 = ((int64_t)blockIdx.x * 64 + tx) * 4;
  const int64_t r0 = (int64_t)blockIdx.y * slab, r_end = r0 + slab < R ? r0 + slab : R;
  uint32_t m[4] = {0u, 0u, 0u, 0u}, mn[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
  bool other = false;
  if (c0 < C) {
#pragma unroll 2
    for (int64_t r = r0 + ty; r < r_end; r += 4) {
      const int64_t i = r * C + c0;
      f4_t w = *reinterpret_cast<const f4_t *>(W + i);
      i4_t ind = {1, 1, 1, 1};
      if (!fix_all)
        ind = *reinterpret_cast<const i4_t *>(I + i);
      w.x = ind.x == 1 ? inq_quantize_value(w.x, p, s_cut) : w.x;
      w.y = ind.y == 1 ? inq_quantize_value(w.y, p, s_cut) : w.y;
      w.z = ind.z == 1 ? inq_quantize_value(w.z, p, s_cut) : w.z;
      w.w = ind.w == 1 ? inq_quantize_value(w.w, p, s_cut) : w.w;
      *reinterpret_cast<f4_t *>(W + i) = w;
      if (fix_all)
        *reinterpret_cast<i4_t *>(I + i) = ind;
      *reinterpret_cast<f4_t *>(old_W + i) = w;
      *reinterpret_cast<i4_t *>(old_I + i) = ind;
      const float v[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t u = __float_as_uint(v[j]) & 0x7fffffffu;
        m[j] = u > m[j] ? u : m[j];
        if (u) {
          mn[j] = u < mn[j] ? u : mn[j];
          other |= (u & 0x007fffffu) != 0u || (u >> 23) == 0u;
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    part[ty][tx * 4 + j] = m[j];
    part_min[ty][tx * 4 + j] = mn[j];
  }
  if (__any(other) && (threadIdx.x & 63) == 0 &&
      __hip_atomic_load(cols.flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
    atomicOr(cols.flag, 1);
  __syncthreads();
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c < C) {
    uint32_t a = max(max(part[0][threadIdx.x], part[1][threadIdx.x]), max(part[2][threadIdx.x], part[3][threadIdx.x]));
    if (a)
      atomicMax(&cols.cmax[c], a);
    a = min(min(part_min[0][threadIdx.x], part_min[1][threadIdx.x]),
            min(part_min[2][threadIdx.x], part_min[3][threadIdx.x]));
    if (a != 0xffffffffu)
      atomicMin(&cols.cmin[c], a);
  }
}

// ---- selection: "largest_abs" (:117-141)
__global__ __launch_bounds__(kBlk) void sel_keys(const float *__restrict__ W, uint32_t *__restrict__ keys,
                                                 uint32_t *__restrict__ vals, int64_t size) {
  for (int64_t i = (int64_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (int64_t)gridDim.x * kBlk) {
    keys[i] = __float_as_uint(W[i]) & 0x7fffffffu;
    vals[i] = (uint32_t)i;
  }
}
__global__ __launch_bounds__(kBlk) void sel_flags_sorted(const int *__restrict__ I, const uint32_t *__restrict__ order,
                                                         int *__restrict__ flags, int64_t size) {
  for (int64_t j = (int64_t)blockIdx.x * kBlk + threadIdx.x; j < size; j += (int64_t)gridDim.x * kBlk)
    flags[j] = (I[order[j]] == 0) ? 1 : 0;
}
// Walks the reference's loop in closed form: with c[j] the number of learnable weights among the first j+1 of the
// sorted order and T = num_learnable / 2, position j is fixed iff it is learnable and c[j] <= T; when T == 0 the
// loop stops after its first iteration, which fixes position 0 if it is learnable.
__global__ __launch_bounds__(kBlk) void sel_mark_sorted(int *__restrict__ I, const uint32_t *__restrict__ order,
                                                        const int *__restrict__ c, int64_t size) {
  const int T = c[size - 1] / 2;
  for (int64_t j = (int64_t)blockIdx.x * kBlk + threadIdx.x; j < size; j += (int64_t)gridDim.x * kBlk) {
    const int before = j ? c[j - 1] : 0;
    const bool learnable = c[j] != before;
    if (learnable && ((T >= 1 && c[j] <= T) || (T == 0 && j == 0)))
      I[order[j]] = 1;
  }
}
// ---- selection: "random" (:143-149)
__global__ __launch_bounds__(kBlk) void sel_flags(const int *__restrict__ I, int *__restrict__ flags, int64_t size) {
  for (int64_t i = (int64_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (int64_t)gridDim.x * kBlk)
    flags[i] = (I[i] == 0) ? 1 : 0;
}
__global__ __launch_bounds__(kBlk) void sel_apply_draws(int *__restrict__ I, const int *__restrict__ c,
                                                        const uint8_t *__restrict__ draws, int64_t size) {
  for (int64_t i = (int64_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (int64_t)gridDim.x * kBlk) {
    const int before = i ? c[i - 1] : 0;
    if (c[i] != before) // learnable: its rank among the learnable weights is `before`
      I[i] = draws[before];
  }
}

unsigned grid_for(int64_t size) {
  int64_t b = ceil_div(size, kBlk);
  return (unsigned)(b > 8192 ? 8192 : (b < 1 ? 1 : b));
}

// `cols` (may be null) with `columns` > 0: W is a [size / columns, columns] matrix about to become a column-scaled
// digit operand; the quantize pass then fills that operand's column statistics and *cols_done is set.
int update_weights(float *W, int *I, float *old_W, int *old_I, int64_t size, int num_bits, int step,
                   nbla_hip_bernoulli_fn draw, void *draw_ctx, int *n1n2_out, void *workspace, size_t workspace_bytes,
                   hipStream_t stream, const ColumnScratch *cols = nullptr, int64_t columns = 0,
                   bool *cols_done = nullptr) {
  if (size <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "INQ weight tensor must not be empty.");
  if (size > 0x7fffffffll)
    return fail(NBLA_HIP_ERR_NOT_IMPLEMENTED, "INQ weight tensors above 2^31 elements are not supported.");
  if (step < 0 || step > 3)
    return fail(NBLA_HIP_ERR_VALUE, "invalid INQ step %d.", step);
  const int selection = step == 2 ? 1 : (step == 3 ? 2 : 0);
  const InqWorkspace ws = plan_inq(size, selection);
  if (workspace_bytes < ws.total || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "INQ workspace too small (%zu < %zu) or misaligned.", workspace_bytes, ws.total);
  if (step == 3 && !draw)
    return fail(NBLA_HIP_ERR_VALUE, "random selection needs a Bernoulli draw callback.");
  int rc = ensure_init();
  if (rc)
    return rc;
  char *base = static_cast<char *>(workspace);
  InqParams *params = reinterpret_cast<InqParams *>(base + ws.params_off);
  uint32_t *partial = reinterpret_cast<uint32_t *>(base + ws.partial_off);
  unsigned nparts = grid_for(size);
  if (nparts > (unsigned)kMaxPartials)
    nparts = kMaxPartials;

  hipLaunchKernelGGL(inq_restore_absmax, dim3(nparts), dim3(kBlk), 0, stream, W, old_W, old_I, size,
                     (aligned16(W) && aligned16(old_W) && aligned16(old_I)) ? 1 : 0, partial);
  NBLA_HIP_LAUNCH_CHECK("inq_restore_absmax");

  if (selection == 1) {
    uint32_t *keys_in = reinterpret_cast<uint32_t *>(base + ws.keys_in_off);
    uint32_t *keys_out = reinterpret_cast<uint32_t *>(base + ws.keys_out_off);
    uint32_t *vals_in = reinterpret_cast<uint32_t *>(base + ws.vals_in_off);
    uint32_t *vals_out = reinterpret_cast<uint32_t *>(base + ws.vals_out_off);
    int *scan = reinterpret_cast<int *>(base + ws.scan_off);
    int *flags = reinterpret_cast<int *>(keys_in); // keys_in is free once the sort has run
    size_t temp_bytes = ws.temp_bytes;
    hipLaunchKernelGGL(sel_keys, dim3(grid_for(size)), dim3(kBlk), 0, stream, W, keys_in, vals_in, size);
    NBLA_HIP_LAUNCH_CHECK("inq selection keys");
    hipError_t e = rocprim::radix_sort_pairs_desc(base + ws.temp_off, temp_bytes, keys_in, keys_out, vals_in, vals_out,
                                                  (size_t)size, 0, 32, stream);
    if (e != hipSuccess)
      return fail_hip(e, "rocprim::radix_sort_pairs_desc");
    hipLaunchKernelGGL(sel_flags_sorted, dim3(grid_for(size)), dim3(kBlk), 0, stream, I, vals_out, flags, size);
    NBLA_HIP_LAUNCH_CHECK("inq selection flags");
    temp_bytes = ws.temp_bytes;
    e = rocprim::inclusive_scan(base + ws.temp_off, temp_bytes, flags, scan, (size_t)size, rocprim::plus<int>(),
                                stream);
    if (e != hipSuccess)
      return fail_hip(e, "rocprim::inclusive_scan");
    hipLaunchKernelGGL(sel_mark_sorted, dim3(grid_for(size)), dim3(kBlk), 0, stream, I, vals_out, scan, size);
    NBLA_HIP_LAUNCH_CHECK("inq selection mark");
  } else if (selection == 2) {
    int *flags = reinterpret_cast<int *>(base + ws.keys_in_off);
    int *scan = reinterpret_cast<int *>(base + ws.scan_off);
    uint8_t *draws = reinterpret_cast<uint8_t *>(base + ws.draws_off);
    size_t temp_bytes = ws.temp_bytes;
    hipLaunchKernelGGL(sel_flags, dim3(grid_for(size)), dim3(kBlk), 0, stream, I, flags, size);
    NBLA_HIP_LAUNCH_CHECK("inq selection flags");
    hipError_t e = rocprim::inclusive_scan(base + ws.temp_off, temp_bytes, flags, scan, (size_t)size,
                                           rocprim::plus<int>(), stream);
    if (e != hipSuccess)
      return fail_hip(e, "rocprim::inclusive_scan");
    // The generator lives on the host (as the reference's std::mt19937 does) and advances by exactly one draw per
    // learnable weight, so their number has to come back first.
    int learnable = 0;
    e = hipMemcpyAsync(&learnable, scan + (size - 1), sizeof(int), hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess)
      e = hipStreamSynchronize(stream);
    if (e != hipSuccess)
      return fail_hip(e, "reading the learnable-weight count");
    if (learnable > 0) {
      std::vector<uint8_t> host(learnable);
      draw(draw_ctx, host.data(), learnable);
      e = hipMemcpyAsync(draws, host.data(), (size_t)learnable, hipMemcpyHostToDevice, stream);
      if (e == hipSuccess)
        e = hipStreamSynchronize(stream); // `host` goes out of scope below
      if (e != hipSuccess)
        return fail_hip(e, "uploading the Bernoulli draws");
      hipLaunchKernelGGL(sel_apply_draws, dim3(grid_for(size)), dim3(kBlk), 0, stream, I, scan, draws, size);
      NBLA_HIP_LAUNCH_CHECK("inq selection apply");
    }
  }

  const int levels = (int)std::pow(2, num_bits - 2); // inq_affine.cpp:165
  const bool with_cols = cols && columns > 0 && columns % 4 == 0 && size % columns == 0 && aligned16(W) &&
                         aligned16(I) && aligned16(old_W) && aligned16(old_I);
  ColumnScratch none;
  none.cmax = none.cmin = nullptr, none.flag = nullptr, none.rows = 0;
  hipLaunchKernelGGL(inq_finalize, dim3(1), dim3(64), 0, stream, partial, (int)nparts, levels,
                     device_cut_table(kCutInqN1), params, with_cols ? *cols : none);
  NBLA_HIP_LAUNCH_CHECK("inq_finalize");
  if (with_cols) {
    const int64_t R = size / columns;
    int slab = 64;
    while (slab < 256 && ceil_div(columns, 256) * ceil_div(R, 2 * slab) >= 1024)
      slab *= 2;
    hipLaunchKernelGGL(inq_quantize_columns, dim3((unsigned)ceil_div(columns, 256), (unsigned)ceil_div(R, slab)),
                       dim3(kBlk), 0, stream, W, I, old_W, old_I, R, columns, slab, step == 1 ? 1 : 0, params,
                       device_cut_table(kCutInqExponent), *cols);
  } else {
    hipLaunchKernelGGL(inq_quantize, dim3(grid_for(size)), dim3(kBlk), 0, stream, W, I, old_W, old_I, size,
                       step == 1 ? 1 : 0, params, device_cut_table(kCutInqExponent));
  }
  NBLA_HIP_LAUNCH_CHECK("inq_quantize");
  if (cols_done)
    *cols_done = with_cols;
  if (n1n2_out) {
    hipError_t e = hipMemcpyAsync(n1n2_out, params, 2 * sizeof(int), hipMemcpyDeviceToDevice, stream);
    if (e != hipSuccess)
      return fail_hip(e, "copying n1/n2");
  }
  return NBLA_HIP_OK;
}

struct ProductWorkspace {
  size_t update_off, split_off, planes_off, flag_off, extra_off, total;
};

// `extra`: further scratch behind the operands (the convolution's channel maxima and split partial results)
ProductWorkspace plan_product(int64_t wsize, int64_t M, int64_t K, int64_t N, int step, size_t extra = 0) {
  ProductWorkspace p;
  size_t off = 0;
  p.update_off = off;
  off += round_up(plan_inq(wsize, step == 2 ? 1 : (step == 3 ? 2 : 0)).total, 256);
  // activations and weights as digit operands
  p.split_off = off;
  off += round_up(nbla_hip_digit_operand_bytes(M, K), 256);
  p.planes_off = off;
  off += round_up(nbla_hip_digit_operand_bytes(N, K), 256);
  p.flag_off = off;
  off += 256;
  p.extra_off = off;
  off += round_up(extra, 256);
  p.total = off;
  return p;
}

// scratch of the convolution product: the unfold's channel maxima (16 slices per input position), then the partial
// results of a split contraction
size_t conv_channel_max_bytes(const ConvGeom &g) {
  return round_up((size_t)16 * g.outer * g.in_sp_size * sizeof(uint32_t), 256);
}
size_t conv_product_extra(const ConvGeom &g) {
  return conv_channel_max_bytes(g) + gemm_digits_split_bytes(g.M, g.Kg, g.Og);
}

} // namespace
} // namespace nbla_hip

using namespace nbla_hip;

extern "C" {

size_t nbla_hip_inq_workspace_bytes(int64_t size, int step) {
  return plan_inq(size, step == 2 ? 1 : (step == 3 ? 2 : 0)).total;
}

int nbla_hip_inq_update_weights_f32(float *W, int32_t *I, float *old_W, int32_t *old_I, int64_t size, int num_bits,
                                    int step, nbla_hip_bernoulli_fn draw, void *draw_ctx, int32_t *n1n2_out,
                                    void *workspace, size_t workspace_bytes, void *stream) {
  return update_weights(W, I, old_W, old_I, size, num_bits, step, draw, draw_ctx, n1n2_out, workspace, workspace_bytes,
                        as_stream(stream));
}

size_t nbla_hip_inq_affine_workspace_bytes(int64_t M, int64_t K, int64_t N, int step) {
  return plan_product(K * N, M, K, N, step, gemm_digits_split_bytes(M, K, N)).total;
}

int nbla_hip_inq_affine_f32(const float *x, float *W, int32_t *I, float *old_W, int32_t *old_I, const float *bias,
                            float *y, int64_t M, int64_t K, int64_t N, int num_bits, int step,
                            nbla_hip_bernoulli_fn draw, void *draw_ctx, void *workspace, size_t workspace_bytes,
                            void *stream_) {
  if (M <= 0 || K <= 0 || N <= 0)
    return fail(NBLA_HIP_ERR_VALUE, "invalid affine shape (M=%lld, K=%lld, N=%lld).", (long long)M, (long long)K,
                (long long)N);
  const ProductWorkspace p = plan_product(K * N, M, K, N, step, gemm_digits_split_bytes(M, K, N));
  if (workspace_bytes < p.total || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "INQ affine workspace too small (%zu < %zu) or misaligned.", workspace_bytes,
                p.total);
  hipStream_t stream = as_stream(stream_);
  char *base = static_cast<char *>(workspace);
  int rc;
  // The product runs on the int8 digit kernels: x as a row-scaled digit operand, W^T as a column-scaled one.  Once
  // every weight is zero or a power of two (all fixed) and a column spans at most six binades, each weight is a small
  // integer in one digit and three exact digit products give the result; otherwise six (weights still being learnt).
  // The weight update's last pass gathers the column statistics of that operand on the way.
  bool cols_done = false;
  if (step >= 0) {
    const ColumnScratch cols = column_scratch(base + p.planes_off, K, N);
    rc = update_weights(W, I, old_W, old_I, K * N, num_bits, step, draw, draw_ctx, nullptr, base + p.update_off,
                        p.split_off - p.update_off, stream, &cols, N, &cols_done);
    if (rc)
      return rc;
  } else {
    rc = ensure_init();
    if (rc)
      return rc;
  }
  rc = nbla_hip_split_digits_f32(x, K, base + p.split_off, M, K, stream_);
  if (rc)
    return rc;
  rc = cols_done ? launch_split_digits_columns_from_stats(W, N, base + p.planes_off, K, N, true, stream)
                 : launch_split_digits_columns(W, N, base + p.planes_off, K, N, true, stream);
  if (rc)
    return rc;
  return launch_gemm_digits(base + p.split_off, base + p.planes_off, bias, y, M, K, N, 1, N, 1, stream, false,
                            base + p.extra_off, gemm_digits_split_bytes(M, K, N));
}

size_t nbla_hip_inq_convolution_workspace_bytes(int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                                const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                                const int64_t *dilation, int64_t group, int step) {
  ConvGeom g;
  if (make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group))
    return 0;
  return plan_product(g.O * g.Kg, g.M, g.Kg, g.Og, step, conv_product_extra(g)).total;
}

int nbla_hip_inq_convolution_f32(const float *x, float *W, int32_t *I, float *old_W, int32_t *old_I, const float *bias,
                                 float *y, int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                 const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                 const int64_t *dilation, int64_t group, int num_bits, int step,
                                 nbla_hip_bernoulli_fn draw, void *draw_ctx, void *workspace, size_t workspace_bytes,
                                 void *stream_) {
  ConvGeom g;
  int rc = make_geom(g, outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group);
  if (rc)
    return rc;
  const ProductWorkspace p = plan_product(g.O * g.Kg, g.M, g.Kg, g.Og, step, conv_product_extra(g));
  if (workspace_bytes < p.total || !aligned256(workspace))
    return fail(NBLA_HIP_ERR_MEMORY, "INQ convolution workspace too small (%zu < %zu) or misaligned.", workspace_bytes,
                p.total);
  hipStream_t stream = as_stream(stream_);
  char *base = static_cast<char *>(workspace);
  if (step >= 0) {
    rc = update_weights(W, I, old_W, old_I, g.O * g.Kg, num_bits, step, draw, draw_ctx, nullptr, base + p.update_off,
                        p.split_off - p.update_off, stream);
    if (rc)
      return rc;
  } else {
    rc = ensure_init();
    if (rc)
      return rc;
  }
  // The product runs on the int8 digit kernels: the unfolded input goes straight into a row-scaled digit operand
  // (rows = output positions), the weights [Og, Kg] into another (rows = output channels); six exact digit products.
  const int64_t hw = g.out_sp_size;
  const size_t cmax_bytes = conv_channel_max_bytes(g);
  for (int64_t grp = 0; grp < g.group; ++grp) {
    rc = launch_im2col_digits(x, base + p.split_off, base + p.extra_off, g, grp, stream);
    if (rc)
      return rc;
    rc = nbla_hip_split_digits_f32(W + grp * g.Og * g.Kg, g.Kg, base + p.planes_off, g.Og, g.Kg, stream_);
    if (rc)
      return rc;
    rc = launch_gemm_digits(base + p.split_off, base + p.planes_off, bias ? bias + grp * g.Og : nullptr,
                            y + grp * g.Og * hw, g.M, g.Kg, g.Og, hw, g.O * hw, hw, stream, false,
                            base + p.extra_off + cmax_bytes, gemm_digits_split_bytes(g.M, g.Kg, g.Og));
    if (rc)
      return rc;
  }
  return NBLA_HIP_OK;
}

size_t nbla_hip_convolution_workspace_bytes(int64_t outer, int64_t C, int nd, const int64_t *in_sp, int64_t O,
                                            const int64_t *kernel, const int64_t *pad, const int64_t *stride,
                                            const int64_t *dilation, int64_t group) {
  return nbla_hip_inq_convolution_workspace_bytes(outer, C, nd, in_sp, O, kernel, pad, stride, dilation, group, -1);
}

// Convolution with real-valued weights: the product-only step of the INQ entry point (the weights are only read).
int nbla_hip_convolution_f32(const float *x, const float *W, const float *bias, float *y, int64_t outer, int64_t C,
                             int nd, const int64_t *in_sp, int64_t O, const int64_t *kernel, const int64_t *pad,
                             const int64_t *stride, const int64_t *dilation, int64_t group, void *workspace,
                             size_t workspace_bytes, void *stream) {
  return nbla_hip_inq_convolution_f32(x, const_cast<float *>(W), nullptr, nullptr, nullptr, bias, y, outer, C, nd, in_sp,
                                      O, kernel, pad, stride, dilation, group, 0, -1, nullptr, nullptr, workspace,
                                      workspace_bytes, stream);
}

} // extern "C"
