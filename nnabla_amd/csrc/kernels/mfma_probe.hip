// Measurement utility (no counterpart in the reference): a kernel of nothing but independent matrix instructions on
// non-zero operands, to read what the matrix pipes of this part sustain under its power limit -- the yardstick the
// product kernels' rates are compared with, and the test of whether another operand format would pay.
//   kind 0: v_mfma_i32_32x32x32_i8 (the instruction of the bit-weight and digit products): 65,536 operations each
//   kind 1: v_mfma_scale_f32_32x32x64_f8f6f4 with fp6 (E2M3) x fp4 (E2M1) operands and unit scales: 131,072 each
//   kind 2: the same instruction with fp8 (E4M3) x fp8 operands
//   kind 3: the int8 instruction with operands that change from one instruction to the next (four random pairs in
//           turn), as in a product where every instruction multiplies new fragments
//   kind 4: as kind 3 with the bit-weight product's operands: random digits against bytes that are 0 or one power
//           of two (a packed word & (0x01010101 << F))
// Every wavefront keeps eight accumulator tiles and issues `rounds` x 8 instructions; the grid is two blocks of four
// wavefronts per CU, like the product kernels.
#include "common.hpp"

namespace nbla_hip {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

template <int kKind> __global__ __launch_bounds__(256, 2) void mfma_rate_kernel(float *sink, int rounds) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t seed = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
  v8i a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (int)((seed >> (i & 3)) * 40503u + 0x9e3779b9u * (i + 1));
    b[i] = (int)((seed << (i & 3)) * 69069u + 0x85ebca6bu * (i + 1));
  }
  float total = 0.0f;
  if (kKind == 3 || kKind == 4) {
    v16i c[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        c[t][r] = 0;
    v4i av[4], bv[4];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[p][i] = (int)((uint32_t)a[i] * (2u * p + 3u) + (uint32_t)b[i + 4] * (2u * p + 1u) + 0x632be5abu * (p + 1));
        const uint32_t w = (uint32_t)b[i] * (2u * p + 5u) + (uint32_t)a[i + 4] + 0x7ed55d16u * (p + 1);
        bv[p][i] = kKind == 4 ? (int)(w & (0x01010101u << (p + i))) : (int)w;
      }
    for (int i = 0; i < rounds; ++i) {
#pragma unroll
      for (int t = 0; t < 8; ++t)
        c[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[t & 3], bv[(t + (t >> 2)) & 3], c[t], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 8; ++t)
      total += (float)c[t][t];
  } else if (kKind == 0) {
    v16i c[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        c[t][r] = 0;
    const v4i a4 = {a[0], a[1], a[2], a[3]}, b4 = {b[0], b[1], b[2], b[3]};
    for (int i = 0; i < rounds; ++i) {
#pragma unroll
      for (int t = 0; t < 8; ++t)
        c[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, b4, c[t], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 8; ++t)
      total += (float)c[t][t];
  } else {
    v16f c[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        c[t][r] = 0.0f;
    if (kKind == 2) { // keep the fp8 operands finite: clear the top exponent bit of every byte
#pragma unroll
      for (int i = 0; i < 8; ++i)
        a[i] &= 0xbfbfbfbf, b[i] &= 0xbfbfbfbf;
    }
    for (int i = 0; i < rounds; ++i) {
#pragma unroll
      for (int t = 0; t < 8; ++t)
        c[t] = kKind == 1 ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c[t], 2, 4, 0, 127, 0, 127)
                          : __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c[t], 0, 0, 0, 127, 0, 127);
    }
#pragma unroll
    for (int t = 0; t < 8; ++t)
      total += c[t][t];
  }
  if (total == 1.2345678f) // never: keeps the accumulators alive without a store per thread
    sink[0] = total;
#endif
}

} // namespace
} // namespace nbla_hip

using namespace nbla_hip;

extern "C" int nbla_hip_mfma_rate_probe(int kind, int rounds, int64_t *instructions, int64_t *ops_per_instruction,
                                         float *sink, void *stream) {
  if (kind < 0 || kind > 4 || rounds < 1 || !sink)
    return fail(NBLA_HIP_ERR_VALUE, "mfma rate probe: kind 0..4, rounds >= 1 and a device word to point at.");
  const int rc = ensure_init();
  if (rc)
    return rc;
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess)
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess)
    return fail_hip(e, "hipDeviceGetAttribute");
  const unsigned blocks = 2u * (unsigned)cus;
  if (kind == 0)
    hipLaunchKernelGGL(mfma_rate_kernel<0>, dim3(blocks), dim3(256), 0, as_stream(stream), sink, rounds);
  else if (kind == 1)
    hipLaunchKernelGGL(mfma_rate_kernel<1>, dim3(blocks), dim3(256), 0, as_stream(stream), sink, rounds);
  else if (kind == 2)
    hipLaunchKernelGGL(mfma_rate_kernel<2>, dim3(blocks), dim3(256), 0, as_stream(stream), sink, rounds);
  else if (kind == 3)
    hipLaunchKernelGGL(mfma_rate_kernel<3>, dim3(blocks), dim3(256), 0, as_stream(stream), sink, rounds);
  else
    hipLaunchKernelGGL(mfma_rate_kernel<4>, dim3(blocks), dim3(256), 0, as_stream(stream), sink, rounds);
  NBLA_HIP_LAUNCH_CHECK("mfma_rate_kernel");
  if (instructions)
    *instructions = (int64_t)blocks * 4 * rounds * 8;
  if (ops_per_instruction)
    *ops_per_instruction = (kind == 0 || kind >= 3) ? 2ll * 32 * 32 * 32 : 2ll * 32 * 32 * 64;
  return NBLA_HIP_OK;
}
