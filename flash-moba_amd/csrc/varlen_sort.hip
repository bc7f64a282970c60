// Segmented ascending sort of signed int32 keys, one workgroup per segment.
//
// LSD radix sort with 8-bit digits.  The byte positions on which all keys of a segment
// agree are skipped (row indices of a 8K-token sequence need two passes, not four).
// Segments of up to kLdsCap keys ping-pong between two LDS buffers and touch HBM exactly
// twice (one read, one write); longer segments ping-pong between the output and a
// caller-provided workspace.  Offsets are 64-bit throughout.
#include "fmoba_common.h"

namespace fmoba {

constexpr int kSortThreads = 256;
constexpr int kLdsCap = 16384;  // keys per LDS buffer (2 x 64 KiB)

__device__ __forceinline__ uint32_t bias_key(int32_t x) { return (uint32_t)x ^ 0x80000000u; }

// One stable counting pass: in[0..n) -> out[0..n) ordered by byte `shift/8`.
// `in`/`out` are generic pointers (LDS or global).  first: input holds raw int32 keys;
// last: output receives raw int32 keys.
__device__ void radix_pass(const uint32_t *in, uint32_t *out, int64_t n, int shift, bool first, bool last, int *hist,
                           int *wsum) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  hist[tid] = 0;
  __syncthreads();
  for (int64_t i = tid; i < n; i += kSortThreads) {
    uint32_t k = in[i];
    if (first) k ^= 0x80000000u;
    atomicAdd(&hist[(k >> shift) & 255u], 1);
  }
  __syncthreads();
  // exclusive scan of the 256 bins (one per thread)
  {
    const int v = hist[tid];
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(incl, o, 64);
      if (lane >= o) incl += t;
    }
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    int add = 0;
    for (int w = 0; w < wave; ++w) add += wsum[w];
    hist[tid] = add + incl - v;
  }
  __syncthreads();
  const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int64_t t0 = 0; t0 < n; t0 += kSortThreads) {
    const int64_t i = t0 + tid;
    const bool valid = i < n;
    uint32_t k = valid ? in[i] : 0u;
    if (first) k ^= 0x80000000u;
    const uint32_t d = (k >> shift) & 255u;
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
      const bool s = (d >> bit) & 1u;
      const unsigned long long bm = __ballot(valid && s);
      peers &= s ? bm : ~bm;
    }
    const int rank = __popcll(peers & lt);
    const int cnt = __popcll(peers);
    int off = 0;
    for (int w = 0; w < kSortThreads / 64; ++w) {
      if (wave == w && valid && rank == 0) {
        off = hist[d];
        hist[d] = off + cnt;
      }
      __syncthreads();
    }
    const int leader = valid ? (__ffsll((long long)peers) - 1) : lane;
    off = __shfl(off, leader, 64);
    if (valid) out[off + rank] = last ? (k ^ 0x80000000u) : k;
  }
  __syncthreads();
}

__global__ __launch_bounds__(kSortThreads) void varlen_sort_kernel(const int64_t *starts, const int64_t *ends, int64_t nseg,
                                                                   const int32_t *src, int32_t *dst, int32_t *tmp, int64_t total) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint32_t *bufA = reinterpret_cast<uint32_t *>(smem);
  uint32_t *bufB = bufA + kLdsCap;
  int *hist = reinterpret_cast<int *>(bufB + kLdsCap);
  int *wsum = hist + 256;
  uint32_t *red = reinterpret_cast<uint32_t *>(wsum + 8);  // [8]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  for (int64_t seg = blockIdx.x; seg < nseg; seg += gridDim.x) {
    const int64_t s = starts[seg], e = ends[seg];
    const int64_t n = e - s;
    if (n <= 0 || s < 0 || e > total) continue;  // uniform
    const uint32_t *in0 = reinterpret_cast<const uint32_t *>(src + s);
    uint32_t *out0 = reinterpret_cast<uint32_t *>(dst + s);
    // range of the biased keys
    uint32_t mn = 0xffffffffu, mx = 0u;
    for (int64_t i = tid; i < n; i += kSortThreads) {
      const uint32_t k = in0[i] ^ 0x80000000u;
      mn = min(mn, k);
      mx = max(mx, k);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      mn = min(mn, (uint32_t)__shfl_xor((int)mn, o, 64));
      mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, 64));
    }
    __syncthreads();
    if (lane == 0) {
      red[wave] = mn;
      red[4 + wave] = mx;
    }
    __syncthreads();
    mn = min(min(red[0], red[1]), min(red[2], red[3]));
    mx = max(max(red[4], red[5]), max(red[6], red[7]));
    const uint32_t diff = mn ^ mx;
    const int passes = diff == 0u ? 0 : (32 - __clz(diff) + 7) / 8;
    if (passes == 0) {
      for (int64_t i = tid; i < n; i += kSortThreads) out0[i] = in0[i];
      __syncthreads();
      continue;
    }
    const bool in_lds = n <= kLdsCap;
    uint32_t *t0 = in_lds ? bufA : out0;
    uint32_t *t1 = in_lds ? bufB : reinterpret_cast<uint32_t *>(tmp + s);
    const uint32_t *cur = in0;
    for (int pi = 0; pi < passes; ++pi) {
      const bool last = pi == passes - 1;
      uint32_t *o;
      if (last)
        o = out0;
      else if (in_lds)
        o = (pi & 1) ? t1 : t0;
      else
        o = ((passes - 1 - pi) & 1) ? t1 : t0;  // alternate so that the last pass lands in dst
      radix_pass(cur, o, n, 8 * pi, pi == 0, last, hist, wsum);
      cur = o;
    }
  }
}

__global__ void fill_zero_i32_kernel(int32_t *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
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
  const size_t smem = (size_t)2 * kLdsCap * 4 + 256 * 4 + 8 * 4 + 8 * 4;
  auto kern = varlen_sort_kernel;
  if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
    set_error("varlen_sort: cannot reserve %zu bytes of LDS", smem);
    return 2;
  }
  const int64_t grid = num_segments < (int64_t)1 << 20 ? num_segments : (int64_t)1 << 20;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kSortThreads), smem, s, seg_starts, seg_ends, num_segments, src, dst,
                     reinterpret_cast<int32_t *>(workspace), total);
  FMOBA_LAUNCH_CHECK("varlen_sort");
  return 0;
}
