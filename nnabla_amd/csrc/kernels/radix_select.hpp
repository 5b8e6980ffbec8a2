// Radix select of the rank-th smallest of up to 2^31 - 1 keys of 31 bits, shared by Prune (keys: the magnitude bits of
// x) and INQ's "largest_abs" selection (keys: the complemented magnitude bits of the learnable weights).
//
// Three passes over the key bits (11, 10, 10), each histogramming the digit of the keys that share the digits chosen
// so far.  A block counts in LDS (four copies of the counters, copy = lane % 4), adds its non-zero counters to one of
// four global copies (a counter that every block of the grid updates is a serial chain of device-wide atomics, 15 ns
// each: the dominant cost with a single copy) and takes a ticket; the block holding the last ticket scans the finished
// histogram and records the chosen digit and the rank left inside it for the next pass.
//
// A kernel of a pass declares the LDS arrays, calls select_begin, feeds every key to select_count and ends with
// select_finish (or, in a chain of launches that each resolve their predecessor's histogram: select_resolve,
// select_begin_at, select_count, select_flush).  The state is cleared by clear_select before pass 0.
#pragma once
#include "common.hpp"

namespace nbla_hip {
namespace {

constexpr int kPasses = 3, kMaxBins = 2048, kLdsCopies = 4, kGlobalCopies = 4;
constexpr int kSelectBlocks = 256;
// 256 histogram blocks of 1024 threads: one per CU; the block that finishes a pass scans the bins with all its
// threads, and fewer blocks mean fewer counter updates (measured against 512 x 256, 512 x 512, 1024 x 512, 512 x 1024)
constexpr int kHistBlock = 1024;
constexpr int kSelectScratch = kHistBlock / 64 + 4; // words of LDS scratch of select_finish / select_resolve
constexpr uint32_t kNoRank = 0xffffffffu; // nothing is to be selected (the passes then leave prefix and rank alone)

struct SelectState {
  uint32_t hist[kPasses][kGlobalCopies][kMaxBins];
  uint32_t done[kPasses];       // blocks of pass p that have added their counters
  uint32_t prefix[kPasses + 1]; // key bits chosen before pass p (entry kPasses: the selected key)
  uint32_t rank[kPasses + 1];   // rank among the keys that share them
  uint32_t count;               // number of keys (written by pass 0)
  uint32_t pad;
  unsigned long long top;       // free for the caller's pass 0 (INQ: the largest magnitude of all and its index)
};
__device__ __forceinline__ int pass_shift(int p) { return p == 0 ? 20 : (p == 1 ? 10 : 0); }
__device__ __forceinline__ int pass_bits(int p) { return p == 0 ? 11 : 10; }

// rank0: the rank to select, or kNoRank when pass 0 derives it from the number of keys (select_finish, kHalf)
__global__ __launch_bounds__(256) void clear_select(SelectState *st, uint32_t rank0) {
  uint32_t *h = &st->hist[0][0][0];
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < kPasses * kGlobalCopies * kMaxBins)
    h[i] = 0u;
  if (i < kPasses)
    st->done[i] = 0u;
  if (i <= kPasses) {
    st->prefix[i] = 0u;
    st->rank[i] = i == 0 ? rank0 : kNoRank;
  }
  if (i == 0) {
    st->count = 0u;
    st->top = 0ull;
  }
}
inline unsigned clear_select_blocks() { return (unsigned)((kPasses * kGlobalCopies * kMaxBins + 255) / 256); }

struct SelectPass {
  uint32_t prefix, rank, mask, want;
  int shift, above, bins, copy, pass;
};

// h: kMaxBins * kLdsCopies words of LDS
__device__ __forceinline__ SelectPass select_begin(uint32_t *h, const SelectState *st, int pass) {
  for (int i = threadIdx.x; i < kMaxBins * kLdsCopies; i += kHistBlock)
    h[i] = 0u;
  SelectPass sp;
  sp.pass = pass;
  sp.prefix = st->prefix[pass], sp.rank = st->rank[pass];
  __syncthreads();
  sp.shift = pass_shift(pass), sp.above = sp.shift + pass_bits(pass), sp.bins = 1 << pass_bits(pass);
  sp.mask = (uint32_t)sp.bins - 1u, sp.want = sp.prefix >> sp.above;
  sp.copy = threadIdx.x & (kLdsCopies - 1);
  return sp;
}

__device__ __forceinline__ void select_count(uint32_t *h, const SelectPass &sp, uint32_t key) {
  if (sp.pass == 0 || (key >> sp.above) == sp.want)
    atomicAdd(&h[((key >> sp.shift) & sp.mask) * kLdsCopies + sp.copy], 1u);
}

// Adds the block's counters to one of the global copies of the pass's histogram.
__device__ __forceinline__ void select_flush(uint32_t *h, SelectState *st, const SelectPass &sp) {
  typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
  __syncthreads();
  uint32_t *g = st->hist[sp.pass][blockIdx.x % kGlobalCopies];
  for (int b = threadIdx.x; b < sp.bins; b += kHistBlock) {
    const uint4_t c = *reinterpret_cast<const uint4_t *>(&h[b * kLdsCopies]);
    const uint32_t total = c.x + c.y + c.z + c.w;
    if (total)
      atomicAdd(&g[b], total);
  }
}

// Scan of the finished histogram of `pass` by one whole block: the digit that holds rank `rank` among the keys sharing
// `prefix`, and the rank inside it.  scratch: kHistBlock / 64 + 4 words of LDS.  Returns through scratch so that every
// thread of the block sees the result: next_prefix, next_rank (kNoRank and prefix unchanged when rank is kNoRank).
// kHalf (pass 0 only): the rank is not given but derived from the number of keys L as L / 2 - 1 (the (L / 2)-th
// smallest), kNoRank when L < 2; thread 0 then also records L in st->count.
struct SelectStep {
  uint32_t prefix, rank;
};
template <bool kHalf>
__device__ __forceinline__ SelectStep select_scan(uint32_t *scratch, SelectState *st, int pass, uint32_t prefix,
                                                  uint32_t rank_in) {
  const int bins = 1 << pass_bits(pass), shift = pass_shift(pass);
  // thread t owns the bins [t * per, (t + 1) * per), per = 2 or 1
  const int per = bins / kHistBlock, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t c[kMaxBins / kHistBlock];
#pragma unroll
  for (int i = 0; i < kMaxBins / kHistBlock; ++i)
    c[i] = 0u;
  for (int k = 0; k < kGlobalCopies; ++k) {
    const unsigned long long *src = reinterpret_cast<const unsigned long long *>(&st->hist[pass][k][threadIdx.x * per]);
    if (per == 1) {
      c[0] += __hip_atomic_load(&st->hist[pass][k][threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      continue;
    }
#pragma unroll
    for (int i = 0; i < kMaxBins / kHistBlock / 2; ++i)
      if (2 * i < per) {
        const unsigned long long two = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        c[2 * i] += (uint32_t)two;
        c[2 * i + 1] += (uint32_t)(two >> 32);
      }
  }
  uint32_t mine = 0;
#pragma unroll
  for (int i = 0; i < kMaxBins / kHistBlock; ++i)
    mine += c[i];
  uint32_t incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off);
    if (lane >= off)
      incl += up;
  }
  if (lane == 63)
    scratch[wave] = incl;
  if (threadIdx.x == 0) {
    scratch[kHistBlock / 64 + 1] = prefix;
    scratch[kHistBlock / 64 + 2] = kNoRank;
  }
  __syncthreads();
  uint32_t excl = incl - mine;
  for (int w = 0; w < wave; ++w)
    excl += scratch[w];
  uint32_t rank = rank_in;
  if (kHalf) {
    uint32_t total = 0;
    for (int w = 0; w < kHistBlock / 64; ++w)
      total += scratch[w];
    rank = total >= 2u ? total / 2u - 1u : kNoRank;
    if (threadIdx.x == 0)
      st->count = total;
  }
  if (rank != kNoRank) {
#pragma unroll
    for (int i = 0; i < kMaxBins / kHistBlock; ++i) {
      if (c[i] != 0u && excl <= rank && rank < excl + c[i]) {
        scratch[kHistBlock / 64 + 1] = prefix | ((uint32_t)(threadIdx.x * per + i) << shift);
        scratch[kHistBlock / 64 + 2] = rank - excl;
      }
      excl += c[i];
    }
  }
  __syncthreads();
  return SelectStep{scratch[kHistBlock / 64 + 1], scratch[kHistBlock / 64 + 2]};
}

// End of a pass whose result the same launch must leave behind: the block that adds its counters last scans the
// finished histogram and records the chosen digit and the rank inside it for the next pass.
// scratch: kHistBlock / 64 + 4 words of LDS.
template <bool kHalf>
__device__ __forceinline__ void select_finish(uint32_t *h, uint32_t *scratch, SelectState *st, const SelectPass &sp) {
  const int pass = sp.pass;
  select_flush(h, st, sp);
  // The ticket must follow this block's counter updates.  A workgroup barrier alone does not order that: it makes no
  // wavefront wait for its own outstanding no-return atomics.  So every wavefront first waits until the memory system
  // has acknowledged all of its vector memory operations (vmcnt(0): a device-scope atomic is acknowledged once it has
  // been performed at the device's coherence point, past the per-XCD L2), then the barrier collects the wavefronts,
  // and only then the ticket is drawn.  Whoever draws the last ticket therefore finds every block's counts in place
  // and reads them with device-scope atomic loads.  No cache write-back or invalidation is involved (the payload is
  // atomics only), which a release / acquire fence per block would cost.
  __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0), expcnt / lgkmcnt untouched
  asm volatile("" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0)
    scratch[kHistBlock / 64] = atomicAdd(&st->done[pass], 1u);
  __syncthreads();
  if (scratch[kHistBlock / 64] != gridDim.x - 1)
    return;
  const SelectStep next = select_scan<kHalf>(scratch, st, pass, sp.prefix, sp.rank);
  if (threadIdx.x == 0 && next.rank != kNoRank) { // else: prefix and rank of the later passes keep their cleared values
    st->prefix[pass + 1] = next.prefix;
    st->rank[pass + 1] = next.rank;
  }
}

// Ticket-free form for a chain of launches: a pass only adds its counters (select_flush); the launch that follows
// resolves the finished histogram itself, every block for itself (2048 bins x 4 copies out of L2), which takes the
// ticket's round trip and the lone last block's scan out of the chain.  Block 0 records what it found for the
// launches after it.  Before pass 0 (and only then) the state's prefix[0] / rank[0] hold the start.
__device__ __forceinline__ SelectStep select_resolve(uint32_t *scratch, SelectState *st, int pass) {
  if (pass == 0)
    return SelectStep{st->prefix[0], st->rank[0]};
  const SelectStep next = select_scan<false>(scratch, st, pass - 1, st->prefix[pass - 1], st->rank[pass - 1]);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    st->prefix[pass] = next.prefix;
    st->rank[pass] = next.rank;
  }
  return next;
}
// select_begin for a pass whose start was found by select_resolve
__device__ __forceinline__ SelectPass select_begin_at(uint32_t *h, const SelectStep &at, int pass) {
  for (int i = threadIdx.x; i < kMaxBins * kLdsCopies; i += kHistBlock)
    h[i] = 0u;
  SelectPass sp;
  sp.pass = pass;
  sp.prefix = at.prefix, sp.rank = at.rank;
  __syncthreads();
  sp.shift = pass_shift(pass), sp.above = sp.shift + pass_bits(pass), sp.bins = 1 << pass_bits(pass);
  sp.mask = (uint32_t)sp.bins - 1u, sp.want = sp.prefix >> sp.above;
  sp.copy = threadIdx.x & (kLdsCopies - 1);
  return sp;
}

} // namespace
} // namespace nbla_hip
