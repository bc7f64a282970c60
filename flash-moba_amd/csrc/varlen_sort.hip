// Segmented ascending sort of signed int32 keys, one workgroup per segment.
//
// LSD radix sort with 8-bit digits.  The byte positions on which all keys of a segment
// agree are skipped (row indices of a 8K-token sequence need two passes, not four).
// A segment of up to kLdsCapMax keys is read into LDS once (the same pass finds the range of
// its keys), ping-pongs between two LDS buffers and is written once: it touches HBM exactly
// twice.  Longer segments ping-pong between the output and a caller-provided workspace.
// Offsets are 64-bit throughout.
//
// Before the radix passes a segment tries the shortcut that row lists allow: keys that do not repeat and span less
// than 32 (64 for the segments that go through HBM) times the buffer size are marked in a bitmap in LDS and enumerated
// in order (bitmap_sort); a repeated key sends the segment to the radix passes.
//
// A counting pass is stable without any order between the waves: every wave owns a contiguous
// block of the keys and a histogram of its own; after the scan, bin d of wave w starts where the
// keys of smaller digits and the digit-d keys of waves before w end.  A wave then walks its block
// 64 keys at a time (lanes with equal digits find each other with eight ballots) and advances
// only its own counters, so the scatter needs no workgroup barrier.
//
// The LDS a workgroup reserves decides how many of them share a compute unit, so segments are
// sorted by size class, one launch per class (2048, 8192, 16384 keys per buffer: seven workgroups of four
// waves, two of eight, one of sixteen per compute unit; the last class also takes the segments that go through HBM).  Every
// launch looks at all segments, 64 at a time with one coalesced load, and takes those of its class.
#include "fmoba_common.h"

namespace fmoba {

constexpr int kLdsCapMax = 16384;  // keys per LDS buffer of the largest class (2 x 64 KiB)

// One stable counting pass over keys [0, n): `load(i)` returns the biased key at position i of the
// input, `store(pos, key)` puts a biased key at its position of the output.  hist: [WAVES][256], wsum: [4].
template <int WAVES, typename Load, typename Store>
__device__ __forceinline__ void radix_pass(Load load, Store store, int64_t n, int shift, int *hist, int *wsum) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t per = ((n + WAVES * 64 - 1) / (WAVES * 64)) * 64;  // keys per wave, a multiple of 64
  const int64_t b0 = min(n, wave * per), b1 = min(n, b0 + per);
  int *myh = hist + wave * 256;
  const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int i = tid; i < WAVES * 256; i += WAVES * 64) hist[i] = 0;
  __syncthreads();
  for (int64_t i = b0 + lane; i < b1; i += 64) atomicAdd(&myh[(load(i) >> shift) & 255u], 1);
  __syncthreads();
  {
    // the first 256 threads, one per bin: exclusive scan of the bin totals, then the waves' shares of the bin in wave order
    int c[WAVES];
    int v = 0, incl = 0;
    if (tid < 256) {
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        c[w] = hist[w * 256 + tid];
        v += c[w];
      }
      incl = v;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
      }
      if (lane == 63) wsum[wave] = incl;
    }
    __syncthreads();
    if (tid < 256) {
      int base = incl - v;
      for (int w = 0; w < wave; ++w) base += wsum[w];
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        hist[w * 256 + tid] = base;
        base += c[w];
      }
    }
  }
  __syncthreads();
  for (int64_t t0 = b0; t0 < b1; t0 += 64) {
    const int64_t i = t0 + lane;
    const bool valid = i < b1;
    const uint32_t k = valid ? load(i) : 0u;
    const uint32_t d = (k >> shift) & 255u;
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
      const bool s = (d >> bit) & 1u;
      const unsigned long long bm = __ballot(valid && s);
      peers &= s ? bm : ~bm;
    }
    const int rank = __popcll(peers & lt);
    int off = 0;
    if (valid && rank == 0) {  // the first lane of each digit advances this wave's counter of the digit
      off = myh[d];
      myh[d] = off + __popcll(peers);
    }
    const int leader = valid ? (__ffsll((long long)peers) - 1) : lane;
    off = __shfl(off, leader, 64);
    if (valid) store(off + rank, k);
  }
  __syncthreads();
}

// Keys that do not repeat and whose range fits a bitmap in LDS need no radix pass: every key sets bit `key - mn`, the
// set bits are counted per thread (a contiguous block of words each), scanned, and enumerated in order.  Returns false,
// with nothing stored, when a key repeats (the caller then runs the radix passes).  `bits` holds nw words, red WAVES.
template <int WAVES, typename Load, typename Store>
__device__ __forceinline__ bool bitmap_sort(Load load, Store store, int64_t n, uint32_t mn, int nw, uint32_t *bits, uint32_t *red) {
  constexpr int kThreads = WAVES * 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < nw; i += kThreads) bits[i] = 0u;
  __syncthreads();
  int dup = 0;
  for (int64_t i = tid; i < n; i += kThreads) {
    const uint32_t b = load(i) - mn;
    const uint32_t m = 1u << (b & 31u);
    dup |= (atomicOr(&bits[b >> 5], m) & m) != 0u;
  }
  if (__syncthreads_or(dup)) return false;
  const int per = (nw + kThreads - 1) / kThreads;
  const int w0 = min(nw, tid * per), w1 = min(nw, w0 + per);
  int cnt = 0;
  for (int w = w0; w < w1; ++w) cnt += __popc(bits[w]);
  int incl = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(incl, o, 64);
    if (lane >= o) incl += t;
  }
  if (lane == 63) red[wave] = (uint32_t)incl;
  __syncthreads();
  int pos = incl - cnt;
  for (int w = 0; w < wave; ++w) pos += (int)red[w];
  for (int w = w0; w < w1; ++w) {
    uint32_t x = bits[w];
    const uint32_t k0 = mn + 32u * (uint32_t)w;
    while (x) {
      store(pos++, k0 + (uint32_t)(__ffs((int)x) - 1));
      x &= x - 1u;
    }
  }
  __syncthreads();
  return true;
}

// range of the biased keys of the workgroup's segment -> number of byte passes (0: all keys equal); mn, mx: the range
template <int WAVES>
__device__ __forceinline__ int radix_passes(uint32_t &mn, uint32_t &mx, uint32_t *red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    mn = min(mn, (uint32_t)__shfl_xor((int)mn, o, 64));
    mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, 64));
  }
  if (lane == 0) {
    red[wave] = mn;
    red[WAVES + wave] = mx;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    mn = min(mn, red[w]);
    mx = max(mx, red[WAVES + w]);
  }
  __syncthreads();  // red is free again
  const uint32_t diff = mn ^ mx;
  return diff == 0u ? 0 : (32 - __clz(diff) + 7) / 8;
}

// Segments of n_lo < n <= n_hi keys: through LDS those of up to CAP keys, through HBM the longer ones (which only the
// last class takes).
// grid: batches of 64 segments x `split` workgroups that share a batch (8 for the smallest class ... 64, i.e. a segment each)
template <int CAP, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void varlen_sort_kernel(const int64_t *starts, const int64_t *ends, int64_t nseg,
                                                                   const int32_t *src, int32_t *dst, int32_t *tmp, int64_t total,
                                                                   int64_t n_lo, int64_t n_hi, int split) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint32_t *bufA = reinterpret_cast<uint32_t *>(smem);
  uint32_t *bufB = bufA + CAP;
  constexpr int kThreads = WAVES * 64;
  int *hist = reinterpret_cast<int *>(bufB + CAP);      // [WAVES][256]
  int *wsum = hist + WAVES * 256;                       // [4]
  uint32_t *red = reinterpret_cast<uint32_t *>(wsum + 4);  // [2 * WAVES]
  const int tid = threadIdx.x, lane = tid & 63;
  const int64_t nbatch = (nseg + 63) / 64;

  // consecutive workgroups share a batch: the segments of one size class come in runs (the first columns of every
  // head are the long ones), and workgroups are dealt to the eight XCDs in turn
  for (int64_t item = blockIdx.x; item < nbatch * split; item += gridDim.x) {
    const int64_t batch = item / split;
    const int part = (int)(item - batch * split);
    // every wave looks at the same 64 segments, so the set of segments to sort is uniform in the workgroup
    const int64_t sg = batch * 64 + lane;
    int64_t s_l = 0, e_l = 0;
    if (sg < nseg) {
      s_l = starts[sg];
      e_l = ends[sg];
    }
    const int64_t n_l = e_l - s_l;
    const bool mine = sg < nseg && n_l > n_lo && n_l <= n_hi && s_l >= 0 && e_l <= total &&
                      (lane % split) == part;
    unsigned long long todo = __ballot(mine);
    while (todo) {
      const int j = __ffsll((long long)todo) - 1;
      todo &= todo - 1;
      const int64_t s = __shfl(s_l, j, 64);
      const int64_t n = __shfl(n_l, j, 64);
      const uint32_t *in0 = reinterpret_cast<const uint32_t *>(src + s);
      uint32_t *out0 = reinterpret_cast<uint32_t *>(dst + s);
      uint32_t mn = 0xffffffffu, mx = 0u;
      if (n <= CAP) {
        for (int i = tid; i < (int)n; i += kThreads) {
          const uint32_t k = in0[i] ^ 0x80000000u;
          bufA[i] = k;
          mn = min(mn, k);
          mx = max(mx, k);
        }
        const int passes = radix_passes<WAVES>(mn, mx, red);
        if (passes == 0) {
          for (int i = tid; i < (int)n; i += kThreads) out0[i] = bufA[i] ^ 0x80000000u;
          __syncthreads();
          continue;
        }
        if ((uint64_t)(mx - mn) < (uint64_t)CAP * 32u) {  // the bitmap fits bufB
          const uint32_t *c = bufA;
          if (bitmap_sort<WAVES>([&](int64_t i) { return c[i]; }, [&](int pos, uint32_t k) { bufA[pos] = k; }, n, mn,
                                 (int)((mx - mn) / 32u) + 1, bufB, red)) {
            for (int i = tid; i < (int)n; i += kThreads) out0[i] = bufA[i] ^ 0x80000000u;
            __syncthreads();
            continue;
          }
        }
        uint32_t *cur = bufA, *oth = bufB;
        for (int pi = 0; pi < passes; ++pi) {
          const uint32_t *c = cur;
          if (pi == passes - 1) {
            radix_pass<WAVES>([&](int64_t i) { return c[i]; }, [&](int pos, uint32_t k) { out0[pos] = k ^ 0x80000000u; }, n, 8 * pi, hist, wsum);
          } else {
            uint32_t *o = oth;
            radix_pass<WAVES>([&](int64_t i) { return c[i]; }, [&](int pos, uint32_t k) { o[pos] = k; }, n, 8 * pi, hist, wsum);
          }
          uint32_t *t = cur;
          cur = oth;
          oth = t;
        }
      } else {
        for (int64_t i = tid; i < n; i += kThreads) {
          const uint32_t k = in0[i] ^ 0x80000000u;
          mn = min(mn, k);
          mx = max(mx, k);
        }
        const int passes = radix_passes<WAVES>(mn, mx, red);
        if (passes == 0) {
          for (int64_t i = tid; i < n; i += kThreads) out0[i] = in0[i];
          __syncthreads();
          continue;
        }
        if ((uint64_t)(mx - mn) < (uint64_t)CAP * 64u) {  // the bitmap fits the two buffers together
          if (bitmap_sort<WAVES>([&](int64_t i) { return in0[i] ^ 0x80000000u; },
                                 [&](int pos, uint32_t k) { out0[pos] = k ^ 0x80000000u; }, n, mn, (int)((mx - mn) / 32u) + 1, bufA, red))
            continue;
        }
        uint32_t *t1 = reinterpret_cast<uint32_t *>(tmp + s);
        const uint32_t *cur = in0;
        for (int pi = 0; pi < passes; ++pi) {
          const bool first = pi == 0, last = pi == passes - 1;
          uint32_t *o = ((passes - 1 - pi) & 1) ? t1 : out0;  // alternate so that the last pass lands in dst
          const uint32_t *c = cur;
          const uint32_t in_bias = first ? 0x80000000u : 0u, out_bias = last ? 0x80000000u : 0u;
          radix_pass<WAVES>([&](int64_t i) { return c[i] ^ in_bias; }, [&](int64_t pos, uint32_t k) { o[pos] = k ^ out_bias; }, n, 8 * pi, hist,
                     wsum);
          cur = o;
        }
      }
    }
  }
}

__global__ void fill_zero_i32_kernel(int32_t *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

template <int CAP, int WAVES>
static int launch_sort_class(const int64_t *seg_starts, const int64_t *seg_ends, int64_t num_segments, const int32_t *src, int32_t *dst,
                             int32_t *tmp, int64_t total, int64_t n_lo, int64_t n_hi, int split, hipStream_t s) {
  const size_t smem = (size_t)2 * CAP * 4 + (size_t)WAVES * 256 * 4 + 4 * 4 + 2 * WAVES * 4;
  auto kern = varlen_sort_kernel<CAP, WAVES>;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("varlen_sort: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int64_t nbatch = (num_segments + 63) / 64;
  const int64_t items = nbatch * split;
  const int64_t grid = items < 4096 ? items : 4096;  // a workgroup takes every 4096th item: few dispatches, and runs of long segments spread out
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(WAVES * 64), smem, s, seg_starts, seg_ends, num_segments, src, dst, tmp, total, n_lo,
                     n_hi, split);
  FMOBA_LAUNCH_CHECK("varlen_sort");
  return 0;
}

}  // namespace fmoba

extern "C" size_t fmoba_varlen_sort_workspace_bytes(int64_t total) { return total > 0 ? (size_t)total * 4 : 0; }

extern "C" int fmoba_varlen_sort(const int64_t *seg_starts, const int64_t *seg_ends, int64_t num_segments, const int32_t *src,
                                 int32_t *dst, int64_t total, void *workspace, size_t workspace_bytes, void *stream) {
  using namespace fmoba;
  FMOBA_REQUIRE(num_segments >= 0 && total >= 0, "varlen_sort: negative size");
  if (total == 0) return 0;
  FMOBA_REQUIRE(src && dst, "varlen_sort: null src/dst");
  FMOBA_REQUIRE(src != dst, "varlen_sort: the sort is out of place (src == dst)");
  FMOBA_REQUIRE(num_segments == 0 || (seg_starts && seg_ends), "varlen_sort: null segment offsets");
  FMOBA_REQUIRE(workspace != nullptr && workspace_bytes >= (size_t)total * 4, "varlen_sort: workspace must hold %lld int32",
                (long long)total);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(fill_zero_i32_kernel, dim3(1024), dim3(256), 0, s, dst, total);
  FMOBA_LAUNCH_CHECK("varlen_sort(zero)");
  if (num_segments == 0) return 0;
  int32_t *tmp = reinterpret_cast<int32_t *>(workspace);
  if (int rc = launch_sort_class<2048, 4>(seg_starts, seg_ends, num_segments, src, dst, tmp, total, 0, 2048, 8, s)) return rc;
  if (total > 2048)
    if (int rc = launch_sort_class<8192, 8>(seg_starts, seg_ends, num_segments, src, dst, tmp, total, 2048, 8192, 32, s)) return rc;
  if (total > 8192)
    if (int rc = launch_sort_class<kLdsCapMax, 16>(seg_starts, seg_ends, num_segments, src, dst, tmp, total, 8192, INT64_MAX, 64, s)) return rc;
  return 0;
}
