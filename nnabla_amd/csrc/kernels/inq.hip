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
#include "radix_select.hpp"
#include "redo_marked.hpp"

#include <cmath>
#include <vector>

namespace nbla_hip {
namespace {

constexpr int kBlk = 256;
constexpr int kMaxPartials = 1024;

struct InqParams {
  int n1, n2;
  float thr;
  int all_fixed; // 1: the snapshot's indicators were all 1 when this call restored the weights
};

// Both selections rank weights in index order inside chunks of whole tiles: one block per chunk, the number of
// ranked weights per chunk in `counts`, turned into each chunk's starting rank by a one-block scan.
constexpr int kSelTile = kBlk * 4;   // weights per block and step: four consecutive ones per thread
constexpr int kMaxChunks = 2048;
struct ChunkPlan {
  int nchunks;
  int64_t chunk; // weights per chunk, a multiple of kSelTile
};
ChunkPlan plan_chunks(int64_t size) {
  ChunkPlan c;
  int64_t n = ceil_div(size, kSelTile);
  if (n > kMaxChunks)
    n = kMaxChunks;
  if (n < 1)
    n = 1;
  c.chunk = ceil_div(ceil_div(size, n), kSelTile) * kSelTile;
  c.nchunks = (int)ceil_div(size, c.chunk);
  return c;
}

struct InqWorkspace {
  size_t params_off, partial_off, state_off, counts_off, draws_off, total;
};

InqWorkspace plan_inq(int64_t size, int selection) {
  InqWorkspace w;
  size_t off = 0;
  w.params_off = off;
  off += 256;
  w.partial_off = off;
  off += round_up(kMaxPartials * sizeof(uint32_t), 256);
  w.state_off = w.counts_off = w.draws_off = off;
  if (selection == 1) { // largest_abs: radix select, then the ties in index order
    w.state_off = off, off += round_up(sizeof(SelectState), 256);
    w.counts_off = off, off += round_up((kMaxChunks + 1) * sizeof(uint32_t), 256);
  } else if (selection == 2) { // random: ranks of the learnable weights + uploaded draws
    w.counts_off = off, off += round_up((kMaxChunks + 1) * sizeof(uint32_t), 256);
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
  bool unfixed = false; // a weight that the snapshot does not hold as fixed
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
      unfixed |= !all0 || !all1;
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
    } else {
      unfixed = true;
    }
    take(w);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const uint32_t o = __shfl_xor(mx, off);
    mx = o > mx ? o : mx;
  }
  // the block's largest magnitude (bit 31 is free: magnitudes), and in bit 31 whether it met an unfixed weight
  mx |= __any(unfixed) ? 0x80000000u : 0u;
  __shared__ uint32_t s_mx[kBlk / 64];
  if ((threadIdx.x & 63) == 0)
    s_mx[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t flag = mx & 0x80000000u;
    mx &= 0x7fffffffu;
    for (int w = 1; w < kBlk / 64; ++w) {
      flag |= s_mx[w] & 0x80000000u;
      mx = (s_mx[w] & 0x7fffffffu) > mx ? (s_mx[w] & 0x7fffffffu) : mx;
    }
    partial[blockIdx.x] = mx | flag;
  }
}

// n1, n2 and the pruning threshold (inq_affine.cpp:157-166).  `levels` is the
// host's (int)pow(2, num_bits - 2).
constexpr int kFinalizeThreads = 1024; // one round trip for the up to kMaxPartials partial maxima
__global__ __launch_bounds__(kFinalizeThreads) void inq_finalize(const uint32_t *__restrict__ partial, int nparts, int levels,
                                                   const uint32_t *__restrict__ n1_cuts, InqParams *__restrict__ params,
                                                   ColumnScratch cols) {
  // the column statistics that the quantize pass will gather (cols.cmax null: none wanted) start from their neutral
  // values
  if (cols.cmax) {
    for (int64_t i = threadIdx.x; i < cols.rows; i += kFinalizeThreads) {
      cols.cmax[i] = 0u;
      cols.cmin[i] = 0xffffffffu;
    }
    if (threadIdx.x == 0)
      *cols.flag = 0;
  }
  uint32_t mx = 0u, unfixed = 0u; // (bit 31 of a partial result: the block met a weight that is not fixed)
  for (int i = threadIdx.x; i < nparts; i += kFinalizeThreads) {
    const uint32_t v = partial[i];
    unfixed |= v >> 31;
    mx = (v & 0x7fffffffu) > mx ? (v & 0x7fffffffu) : mx;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const uint32_t o = __shfl_xor(mx, off);
    mx = o > mx ? o : mx;
  }
  mx |= __any(unfixed != 0u) ? 0x80000000u : 0u;
  __shared__ uint32_t s_mx[kFinalizeThreads / 64];
  if ((threadIdx.x & 63) == 0)
    s_mx[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x != 0)
    return;
  unfixed = mx >> 31;
  mx &= 0x7fffffffu;
  for (int w = 1; w < kFinalizeThreads / 64; ++w) {
    unfixed |= s_mx[w] >> 31;
    mx = (s_mx[w] & 0x7fffffffu) > mx ? (s_mx[w] & 0x7fffffffu) : mx;
  }
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
  p.all_fixed = unfixed ? 0 : 1;
  *params = p;
}

// Step C for one fixed weight (:168-190).
__device__ __forceinline__ float inq_quantize_value(float w, const InqParams &p, const uint32_t *s_cut) {
  const uint32_t u = __float_as_uint(w) & 0x7fffffffu;
  // A weight that is already one of the levels -- a normal power of two with exponent in [n2, n1] -- comes back as
  // it is: it lies above the pruning threshold 2^(n2 - 1), below the cut of its own binade, inside the clamp.  That
  // is every weight but the zeros once quantized weights are quantized again (all of them, every forward, when all
  // are fixed), and it spares them the table look-up.
  const int eb = (int)(u >> 23) - 127;
  if ((u & 0x007fffffu) == 0u && eb >= p.n2 && eb <= p.n1 && eb > -127 && eb <= 127)
    return w;
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
  const bool settled = p.all_fixed != 0 && !fix_all;
  for (int64_t i = (int64_t)blockIdx.x * kBlk + threadIdx.x; i < size; i += (int64_t)gridDim.x * kBlk) {
    const float w0 = W[i];
    float w = w0;
    const int ind = fix_all ? 1 : I[i];
    if (ind == 1)
      w = inq_quantize_value(w, p, s_cut);
    // A fixed weight of a snapshot that held every weight as fixed was copied from that snapshot by this call's
    // restoring pass; if quantizing leaves its bits alone, W, the snapshot and its indicator hold the values
    // already and nothing is written (the steady state once every weight is fixed).
    if (settled && ind == 1 && __float_as_uint(w) == __float_as_uint(w0))
      continue;
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
  const bool settled = p.all_fixed != 0 && !fix_all;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int64_t c0 = ((int64_t)blockIdx.x * 64 + tx) * 4;
  const int64_t r0 = (int64_t)blockIdx.y * slab, r_end = r0 + slab < R ? r0 + slab : R;
  uint32_t m[4] = {0u, 0u, 0u, 0u}, mn[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
  bool other = false;
  if (c0 < C) {
#pragma unroll 2
    for (int64_t r = r0 + ty; r < r_end; r += 4) {
      const int64_t i = r * C + c0;
      const f4_t w0 = *reinterpret_cast<const f4_t *>(W + i);
      f4_t w = w0;
      i4_t ind = {1, 1, 1, 1};
      if (!fix_all)
        ind = *reinterpret_cast<const i4_t *>(I + i);
      w.x = ind.x == 1 ? inq_quantize_value(w.x, p, s_cut) : w.x;
      w.y = ind.y == 1 ? inq_quantize_value(w.y, p, s_cut) : w.y;
      w.z = ind.z == 1 ? inq_quantize_value(w.z, p, s_cut) : w.z;
      w.w = ind.w == 1 ? inq_quantize_value(w.w, p, s_cut) : w.w;
      // (see inq_quantize: nothing to write where the snapshot already holds these four fixed weights)
      const bool same = settled && ind.x == 1 && ind.y == 1 && ind.z == 1 && ind.w == 1 &&
                        __float_as_uint(w.x) == __float_as_uint(w0.x) && __float_as_uint(w.y) == __float_as_uint(w0.y) &&
                        __float_as_uint(w.z) == __float_as_uint(w0.z) && __float_as_uint(w.w) == __float_as_uint(w0.w);
      if (!same) {
        *reinterpret_cast<f4_t *>(W + i) = w;
        if (fix_all)
          *reinterpret_cast<i4_t *>(I + i) = ind;
        *reinterpret_cast<f4_t *>(old_W + i) = w;
        *reinterpret_cast<i4_t *>(old_I + i) = ind;
      }
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
// The reference sorts all indices by falling |w| and then fixes learnable weights in that order until T =
// num_learnable / 2 of them are fixed: the T learnable weights of largest magnitude.  Here: a radix select over the
// learnable weights finds the T-th largest magnitude t (keys are the complemented magnitude bits, so "largest" is
// "smallest key"; a NaN orders above every number, as its bits do) and how many of the weights of magnitude exactly t
// belong to the T; those are taken in index order (the order a stable sort gives; the reference's std::sort leaves
// the order of equal magnitudes to the library).  When T == 0 the reference's loop still runs once: it fixes the
// first index of the sorted order, whatever its magnitude rank among learnable weights, if that one is learnable.
__device__ __forceinline__ uint32_t inq_key(float w) { return 0x7fffffffu - (__float_as_uint(w) & 0x7fffffffu); }

__global__ __launch_bounds__(kHistBlock) void inq_select_histogram(const float *__restrict__ W,
                                                                   const int *__restrict__ I, int64_t n4, int64_t n,
                                                                   SelectState *__restrict__ st, int pass) {
  typedef float f4_t __attribute__((ext_vector_type(4)));
  typedef int i4_t __attribute__((ext_vector_type(4)));
  __shared__ uint32_t h[kMaxBins * kLdsCopies];
  __shared__ uint32_t scratch[kSelectScratch];
  const SelectPass sp = select_begin(h, st, pass);
  // pass 0 also finds the first index of the sorted order: the largest magnitude of all weights, lowest index first
  unsigned long long top = 0ull;
  auto count = [&](float w, int ind, int64_t i) {
    const uint32_t key = inq_key(w);
    if (ind == 0)
      select_count(h, sp, key);
    if (pass == 0) {
      const unsigned long long cand =
          ((unsigned long long)(0x7fffffffu - key) << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
      top = cand > top ? cand : top;
    }
  };
  const int64_t tiles = (n4 + kHistBlock * 2 - 1) / (kHistBlock * 2);
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t base = tile * (kHistBlock * 2) + threadIdx.x;
    f4_t v[2];
    i4_t f[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
      if (base + j * kHistBlock < n4) {
        v[j] = reinterpret_cast<const f4_t *>(W)[base + j * kHistBlock];
        f[j] = reinterpret_cast<const i4_t *>(I)[base + j * kHistBlock];
      }
#pragma unroll
    for (int j = 0; j < 2; ++j)
      if (base + j * kHistBlock < n4) {
        const int64_t i = 4 * (base + j * kHistBlock);
        count(v[j].x, f[j].x, i), count(v[j].y, f[j].y, i + 1), count(v[j].z, f[j].z, i + 2),
            count(v[j].w, f[j].w, i + 3);
      }
  }
  // what the 16-byte accesses leave: up to three weights, or all of them when the arrays are not aligned
  for (int64_t i = 4 * n4 + (int64_t)blockIdx.x * kHistBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kHistBlock)
    count(W[i], I[i], i);
  if (pass == 0) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const unsigned long long o = __shfl_xor(top, off);
      top = o > top ? o : top;
    }
    if ((threadIdx.x & 63) == 0 && top != 0ull)
      atomicMax(&st->top, top);
    select_finish<true>(h, scratch, st, sp);
  } else {
    select_finish<false>(h, scratch, st, sp);
  }
}

// What a selection ranks: kTies -- the learnable weights of the selected magnitude; otherwise every learnable weight.
template <bool kTies>
__device__ __forceinline__ uint32_t sel_ranked(const float *__restrict__ W, const int *__restrict__ I, int64_t i,
                                               int64_t size, uint32_t key) {
  if (i >= size || I[i] != 0)
    return 0u;
  return kTies ? (inq_key(W[i]) == key ? 1u : 0u) : 1u;
}

template <bool kTies>
__global__ __launch_bounds__(kBlk) void sel_count_chunks(const float *__restrict__ W, const int *__restrict__ I,
                                                         int64_t size, int64_t chunk,
                                                         const SelectState *__restrict__ st,
                                                         uint32_t *__restrict__ counts) {
  uint32_t key = 0u;
  if (kTies) {
    if (st->rank[kPasses] == kNoRank) { // nothing to rank
      if (threadIdx.x == 0)
        counts[blockIdx.x] = 0u;
      return;
    }
    key = st->prefix[kPasses];
  }
  const int64_t begin = (int64_t)blockIdx.x * chunk;
  uint32_t c = 0u;
  for (int64_t t = begin; t < begin + chunk && t < size; t += kSelTile)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      c += sel_ranked<kTies>(W, I, t + j * kBlk + threadIdx.x, size, key);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1)
    c += __shfl_xor(c, off);
  __shared__ uint32_t s_part[kBlk / 64];
  if ((threadIdx.x & 63) == 0)
    s_part[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kBlk / 64; ++w)
      c += s_part[w];
    counts[blockIdx.x] = c;
  }
}

// counts[0 .. n) -> exclusive prefix sums in place, the total in counts[n]
__global__ __launch_bounds__(kBlk) void sel_scan_counts(uint32_t *__restrict__ counts, int n) {
  __shared__ uint32_t s_wave[kBlk / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t carry = 0u;
  for (int base = 0; base < n; base += kBlk) {
    const int i = base + threadIdx.x;
    const uint32_t v = i < n ? counts[i] : 0u;
    uint32_t incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off);
      if (lane >= off)
        incl += up;
    }
    __syncthreads(); // the previous step's s_wave has been read
    if (lane == 63)
      s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = carry, total = 0u;
    for (int w = 0; w < kBlk / 64; ++w) {
      before += w < wave ? s_wave[w] : 0u;
      total += s_wave[w];
    }
    if (i < n)
      counts[i] = before + incl - v;
    carry += total;
  }
  if (threadIdx.x == 0)
    counts[n] = carry;
}

// Walks a chunk in index order handing every ranked weight its rank (its number among all ranked weights before it);
// thread t of a step owns the four consecutive weights 4 t .. 4 t + 3 of the step's tile.
template <bool kTies, class Apply>
__device__ __forceinline__ void sel_walk_ranks(const float *__restrict__ W, const int *__restrict__ I, int64_t size,
                                               int64_t chunk, uint32_t key, uint32_t start, Apply apply) {
  __shared__ uint32_t s_wave[kBlk / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t begin = (int64_t)blockIdx.x * chunk;
  uint32_t carry = start;
  for (int64_t t = begin; t < begin + chunk && t < size; t += kSelTile) {
    const int64_t i0 = t + 4 * threadIdx.x;
    uint32_t f[4], mine = 0u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[j] = sel_ranked<kTies>(W, I, i0 + j, size, key);
      mine += f[j];
    }
    uint32_t incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off);
      if (lane >= off)
        incl += up;
    }
    __syncthreads();
    if (lane == 63)
      s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = carry, total = 0u;
    for (int w = 0; w < kBlk / 64; ++w) {
      before += w < wave ? s_wave[w] : 0u;
      total += s_wave[w];
    }
    uint32_t r = before + incl - mine;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      apply(i0 + j, f[j] != 0u, r);
      r += f[j];
    }
    carry += total;
  }
}

__global__ __launch_bounds__(kBlk) void sel_mark_largest(const float *__restrict__ W, int *__restrict__ I, int64_t size,
                                                         int64_t chunk, const SelectState *__restrict__ st,
                                                         const uint32_t *__restrict__ starts) {
  const uint32_t key = st->prefix[kPasses], last = st->rank[kPasses];
  if (last == kNoRank) { // T == 0: only the first index of the sorted order is looked at
    if (blockIdx.x == 0 && threadIdx.x == 0 && st->top != 0ull) {
      const uint32_t i = 0xffffffffu - (uint32_t)st->top;
      if (I[i] == 0)
        I[i] = 1;
    }
    return;
  }
  sel_walk_ranks<true>(W, I, size, chunk, key, starts[blockIdx.x], [&](int64_t i, bool tie, uint32_t r) {
    if (i >= size || I[i] != 0)
      return;
    if (inq_key(W[i]) < key || (tie && r <= last))
      I[i] = 1;
  });
}

// ---- selection: "random" (:143-149): learnable weight number r (in index order) takes draw r
__global__ __launch_bounds__(kBlk) void sel_apply_draws(int *__restrict__ I, int64_t size, int64_t chunk,
                                                        const uint32_t *__restrict__ starts,
                                                        const uint8_t *__restrict__ draws) {
  sel_walk_ranks<false>(nullptr, I, size, chunk, 0u, starts[blockIdx.x], [&](int64_t i, bool learnable, uint32_t r) {
    if (learnable)
      I[i] = draws[r];
  });
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

  const ChunkPlan cp = plan_chunks(size);
  uint32_t *counts = reinterpret_cast<uint32_t *>(base + ws.counts_off);
  if (selection == 1) {
    SelectState *st = reinterpret_cast<SelectState *>(base + ws.state_off);
    const bool vec = aligned16(W) && aligned16(I);
    const int64_t n4 = vec ? size / 4 : 0;
    int64_t blocks = vec ? ceil_div(n4 ? n4 : 1, (int64_t)kHistBlock * 2) : ceil_div(size, (int64_t)kHistBlock);
    if (blocks > kSelectBlocks)
      blocks = kSelectBlocks;
    hipLaunchKernelGGL(clear_select, dim3(clear_select_blocks()), dim3(256), 0, stream, st, kNoRank);
    NBLA_HIP_LAUNCH_CHECK("inq selection clear");
    for (int p = 0; p < kPasses; ++p) {
      hipLaunchKernelGGL(inq_select_histogram, dim3((unsigned)blocks), dim3(kHistBlock), 0, stream, W, I, n4, size, st,
                         p);
      NBLA_HIP_LAUNCH_CHECK("inq selection histogram");
    }
    hipLaunchKernelGGL(sel_count_chunks<true>, dim3((unsigned)cp.nchunks), dim3(kBlk), 0, stream, W, I, size, cp.chunk,
                       st, counts);
    NBLA_HIP_LAUNCH_CHECK("inq selection tie counts");
    hipLaunchKernelGGL(sel_scan_counts, dim3(1), dim3(kBlk), 0, stream, counts, cp.nchunks);
    NBLA_HIP_LAUNCH_CHECK("inq selection scan");
    hipLaunchKernelGGL(sel_mark_largest, dim3((unsigned)cp.nchunks), dim3(kBlk), 0, stream, W, I, size, cp.chunk, st,
                       counts);
    NBLA_HIP_LAUNCH_CHECK("inq selection mark");
  } else if (selection == 2) {
    uint8_t *draws = reinterpret_cast<uint8_t *>(base + ws.draws_off);
    hipLaunchKernelGGL(sel_count_chunks<false>, dim3((unsigned)cp.nchunks), dim3(kBlk), 0, stream, nullptr, I, size,
                       cp.chunk, nullptr, counts);
    NBLA_HIP_LAUNCH_CHECK("inq selection counts");
    hipLaunchKernelGGL(sel_scan_counts, dim3(1), dim3(kBlk), 0, stream, counts, cp.nchunks);
    NBLA_HIP_LAUNCH_CHECK("inq selection scan");
    // The generator lives on the host (as the reference's std::mt19937 does) and advances by exactly one draw per
    // learnable weight, so their number has to come back first.
    int learnable = 0;
    hipError_t e = hipMemcpyAsync(&learnable, counts + cp.nchunks, sizeof(int), hipMemcpyDeviceToHost, stream);
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
      hipLaunchKernelGGL(sel_apply_draws, dim3((unsigned)cp.nchunks), dim3(kBlk), 0, stream, I, size, cp.chunk, counts,
                         draws);
      NBLA_HIP_LAUNCH_CHECK("inq selection apply");
    }
  }

  const int levels = (int)std::pow(2, num_bits - 2); // inq_affine.cpp:165
  const bool with_cols = cols && columns > 0 && columns % 4 == 0 && size % columns == 0 && aligned16(W) &&
                         aligned16(I) && aligned16(old_W) && aligned16(old_I);
  ColumnScratch none;
  none.cmax = none.cmin = nullptr, none.flag = nullptr, none.rows = 0;
  hipLaunchKernelGGL(inq_finalize, dim3(1), dim3(kFinalizeThreads), 0, stream, partial, (int)nparts, levels,
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
  // a handful of rows: one fp32 pass over W instead of its conversion to a digit operand (the split operand's and
  // the weights' operand's space holds the partial results)
  if (affine_few_rows_applies(x, W, y, M, K, N) &&
      p.flag_off - p.split_off >= affine_few_rows_workspace_bytes(M, K, N))
    return launch_affine_few_rows(x, W, bias, y, M, K, N, base + p.split_off, p.flag_off - p.split_off, stream);
  rc = nbla_hip_split_digits_f32(x, K, base + p.split_off, M, K, stream_);
  if (rc)
    return rc;
  rc = cols_done ? launch_split_digits_columns_from_stats(W, N, base + p.planes_off, K, N, true, stream)
                 : launch_split_digits_columns(W, N, base + p.planes_off, K, N, true, stream);
  if (rc)
    return rc;
  rc = launch_gemm_digits(base + p.split_off, base + p.planes_off, bias, y, M, K, N, 1, N, 1, stream, false,
                          base + p.extra_off, gemm_digits_split_bytes(M, K, N));
  if (rc)
    return rc;
  // rows of x and columns of W holding a NaN or an infinity: their outputs one by one, as affine.cpp:87-95 gives them
  return launch_product_redo(DenseRows{x, K}, W, N, 1, bias, y, 1, N, 1, base + p.split_off, base + p.planes_off, M, K,
                             N, stream);
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
  if (conv_direct_forward_applies(g)) // many small groups: all of them in one fp32 launch
    return launch_conv_direct_forward(x, W, nullptr, bias, y, g, stream);
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
    // windows of x and output channels of W holding a NaN or an infinity: their outputs one by one
    // (convolution.cpp:185-193)
    rc = launch_product_redo(UnfoldedRows{x, g, grp}, W + grp * g.Og * g.Kg, 1, g.Kg,
                             bias ? bias + grp * g.Og : nullptr, y + grp * g.Og * hw, hw, g.O * hw, hw,
                             base + p.split_off, base + p.planes_off, g.M, g.Kg, g.Og, stream);
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
